"""``torch.library`` operators for the fused convolution / batch-norm / LIF chains, so that a tracing compiler
(``torch.compile``) keeps them: schema, fake kernels and registered backward formulas around the launch helpers of
``conv_bn_lif.py`` and ``attention_kernel.py``.  Eager calls keep the ``autograd.Function`` s of those modules (the same
helpers, less dispatch overhead); results are identical.

    sj::hip_bn_lif_forward / _backward                 batch norm + LIF over a convolution output
    sj::hip_conv_bn_lif_forward / _backward            Conv(k=1) + batch norm + LIF; with heads > 0 the spikes are
                                                       bit-packed and the output is the contraction scale (V K^T) Q
    sj::hip_lif_conv_bn_lif_forward / _backward        LIF (spikes as bits) + Conv(k=1) + batch norm + LIF
    sj::hip_lif_ssa_forward / _backward                LIF (spikes as bits) + contraction

The reference's kernel backends are compile-transparent custom operators of the same kind
(``cuda_kernel/neuron_kernel/multi_step/lif.py:144-225``; ``test/activation_based/test_compile_compat.py:125-170``).
Optional tensors that an operator does not return are empty tensors (a schema has no optional returns).  An operator
with a backward formula must not write to its arguments: the forward operators return the updated running statistics
and the wrappers below copy them into the module's buffers and count the batch (two small copies and an increment that
the eager path's kernels do on the way).
"""

from __future__ import annotations

from typing import Optional

import torch

from . import attention_kernel as A
from . import conv_bn_lif as C
from . import library as L
from . import neuron_kernel as K

__all__ = ["bn_lif", "conv_bn_lif", "lif_conv_bn_lif", "lif_ssa"]


def _e(ref: torch.Tensor) -> torch.Tensor:
    return ref.new_empty((0,))


def _or_empty(t: Optional[torch.Tensor], ref: torch.Tensor) -> torch.Tensor:
    return t if t is not None else _e(ref)


def _none_if_empty(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    return None if t is None or t.numel() == 0 else t


def _updated(batch_stats: bool, running_mean, running_var):
    """Copies of the running statistics for the launch that updates them in place, or the tensors themselves when they
    are only read (evaluation) or absent."""
    if batch_stats and running_mean is not None and running_var is not None:
        return running_mean.clone(), running_var.clone(), True
    return running_mean, running_var, False


def _write_back(bn, new_mean, new_var) -> None:
    running_mean, running_var, batch_stats, _, _, tracked = C._bn_config(bn)
    with torch.no_grad():  # (the operator's outputs hang on its autograd node: the buffers must not)
        if batch_stats and running_mean is not None and running_var is not None:
            running_mean.copy_(new_mean.detach())
            running_var.copy_(new_var.detach())
        if tracked is not None:
            tracked.add_(1)


# =================================================================================================
# batch norm + LIF
# =================================================================================================
@torch.library.custom_op("sj::hip_bn_lif_forward", mutates_args=())
def hip_bn_lif_forward(y: torch.Tensor, gamma: Optional[torch.Tensor], beta: Optional[torch.Tensor], v_init: torch.Tensor,
                       running_mean: Optional[torch.Tensor], running_var: Optional[torch.Tensor], batch_stats: bool,
                       momentum: float, eps: float, tau: float, v_th: float, v_reset: float, flags: int, sg_id: int,
                       sg_alpha: float, k: Optional[torch.Tensor] = None
                       ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(spikes, v_last, bn_map, new running mean, new running variance)`` (the last two empty when not updated).
    ``k``: ``sigmoid(w)`` of a parametric LIF, one element (``tau`` is then unused)."""
    spec = (tau, v_th, v_reset, flags, sg_id, sg_alpha)
    rm, rv, upd = _updated(batch_stats, running_mean, running_var)
    spikes, v_last, bn_map = C._BnLif.forward(y, gamma, beta, v_init, (rm, rv, batch_stats, momentum, eps, None), spec, k)
    return spikes, v_last, bn_map, rm if upd else _e(y), rv if upd else _e(y)


def _fake_running(ref, batch_stats, running_mean, running_var):
    upd = batch_stats and running_mean is not None and running_var is not None
    return (torch.empty_like(running_mean) if upd else _e(ref), torch.empty_like(running_var) if upd else _e(ref))


@hip_bn_lif_forward.register_fake
def _(y, gamma, beta, v_init, running_mean, running_var, batch_stats, momentum, eps, tau, v_th, v_reset, flags, sg_id, sg_alpha,
      k=None):
    T, B, Cc, Lp = y.shape
    return (torch.empty_like(y), y.new_empty((B, Cc, Lp)), y.new_empty((4, Cc)),
            *_fake_running(y, batch_stats, running_mean, running_var))


@torch.library.custom_op("sj::hip_bn_lif_backward", mutates_args=())
def hip_bn_lif_backward(grad_spikes: Optional[torch.Tensor], grad_v_last: Optional[torch.Tensor], y: torch.Tensor,
                        gamma: Optional[torch.Tensor], v_init: torch.Tensor, bn_map: torch.Tensor, batch_stats: bool,
                        tau: float, v_th: float, v_reset: float, flags: int, sg_id: int, sg_alpha: float,
                        need_gvi: bool, k: Optional[torch.Tensor] = None
                        ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(dy, dgamma, dbeta, grad_v_init or empty, dL/dk or empty)``."""
    spec = (tau, v_th, v_reset, flags, sg_id, sg_alpha)
    dy, dgamma, dbeta, gvi, *grad_k = C._bn_lif_backward(L.aligned16(y), bn_map, gamma, v_init, spec, batch_stats, grad_spikes,
                                                         grad_v_last, need_gvi, False, k)
    # (dgamma and dbeta are rows of one buffer)
    return dy, dgamma.clone(), dbeta.clone(), _or_empty(gvi, y), grad_k[0] if grad_k else _e(y)


@hip_bn_lif_backward.register_fake
def _(grad_spikes, grad_v_last, y, gamma, v_init, bn_map, batch_stats, tau, v_th, v_reset, flags, sg_id, sg_alpha, need_gvi,
      k=None):
    T, B, Cc, Lp = y.shape
    return (torch.empty_like(y), y.new_empty((Cc,)), y.new_empty((Cc,)), y.new_empty((B, Cc, Lp) if need_gvi else (0,)),
            y.new_empty((1,) if k is not None else (0,)))


def _bn_lif_setup(ctx, inputs, output):
    (y, gamma, beta, v_init, running_mean, running_var, batch_stats, momentum, eps, tau, v_th, v_reset, flags, sg_id,
     sg_alpha, k) = inputs
    ctx.scalars = (batch_stats, tau, v_th, v_reset, flags, sg_id, sg_alpha)
    ctx.has_gamma = gamma is not None
    ctx.save_for_backward(y, gamma, v_init, output[2], k)
    ctx.set_materialize_grads(False)


def _bn_lif_formula(ctx, grad_spikes, grad_v_last, grad_map, _rm, _rv):
    del grad_map
    y, gamma, v_init, bn_map, k = ctx.saved_tensors
    need = ctx.needs_input_grad
    dy, dgamma, dbeta, gvi, grad_k = hip_bn_lif_backward(grad_spikes, grad_v_last, y, gamma, v_init, bn_map, *ctx.scalars,
                                                         bool(need[3]), k)
    return (dy if need[0] else None, dgamma if need[1] else None, dbeta if need[2] else None, gvi if need[3] else None) + \
        (None,) * 11 + (grad_k if k is not None and need[15] else None,)


torch.library.register_autograd("sj::hip_bn_lif_forward", _bn_lif_formula, setup_context=_bn_lif_setup)


def bn_lif(y_seq, gamma, beta, v_init, bn, spec, k=None):
    running_mean, running_var, batch_stats, momentum, eps, _ = C._bn_config(bn)
    spikes, v_last, _, new_mean, new_var = hip_bn_lif_forward(y_seq, gamma, beta, v_init, running_mean, running_var, batch_stats,
                                                              momentum, eps, *spec, k)
    _write_back(bn, new_mean, new_var)
    return spikes, v_last


# =================================================================================================
# convolution + batch norm + LIF (+ contraction)
# =================================================================================================
def _packed_bytes(T, B, Cout, Lp):
    return T * B * Cout * Lp // 8


@torch.library.custom_op("sj::hip_conv_bn_lif_forward", mutates_args=())
def hip_conv_bn_lif_forward(x_seq: torch.Tensor, weight: torch.Tensor, gamma: Optional[torch.Tensor],
                            beta: Optional[torch.Tensor], v_init: torch.Tensor, running_mean: Optional[torch.Tensor],
                            running_var: Optional[torch.Tensor], batch_stats: bool, momentum: float, eps: float, tau: float,
                            v_th: float, v_reset: float, flags: int, sg_id: int, sg_alpha: float, x_exact: bool, terms: int,
                            heads: int, cph: int, scale: float, k: Optional[torch.Tensor] = None
                            ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                                       torch.Tensor, torch.Tensor]:
    """``(out, v_last, y, bn_map, bits, x_amax, new running mean, new running variance)``: ``out`` is the dense spikes
    ``[T, B, Cout, L]`` (``heads == 0``; no bits) or ``scale (V K^T) Q [T * B, heads, cph, L]`` of the bit-packed spikes."""
    if terms != C._terms():
        raise RuntimeError("configure.hip_conv_split / hip_conv_terms changed after this call was compiled")
    spec = (tau, v_th, v_reset, flags, sg_id, sg_alpha)
    rm, rv, upd = _updated(batch_stats, running_mean, running_var)
    bn = (rm, rv, batch_stats, momentum, eps, None)
    new = (rm if upd else _e(x_seq), rv if upd else _e(x_seq))
    if heads == 0:
        spikes, v_last, y, bn_map, x_amax = C._ConvBnLif.forward(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, k)
        return (spikes, v_last, y, bn_map, torch.empty((0,), dtype=torch.uint8, device=x_seq.device), x_amax, *new)
    return (*C._ConvBnLifSsa.forward(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, (heads, cph, scale), k), *new)


@hip_conv_bn_lif_forward.register_fake
def _(x_seq, weight, gamma, beta, v_init, running_mean, running_var, batch_stats, momentum, eps, tau, v_th, v_reset,
      flags, sg_id, sg_alpha, x_exact, terms, heads, cph, scale, k=None):
    T, B, _, Lp = x_seq.shape
    Cout = weight.shape[0]
    out = x_seq.new_empty((T, B, Cout, Lp) if heads == 0 else (T * B, heads, cph, Lp))
    bits = torch.empty((0 if heads == 0 else _packed_bytes(T, B, Cout, Lp),), dtype=torch.uint8, device=x_seq.device)
    x_amax = x_seq.new_empty((C.amax_floats(T * B) if (terms & C.F16) and not x_exact else 0,))
    return (out, x_seq.new_empty((B, Cout, Lp)), x_seq.new_empty((T, B, Cout, Lp)), x_seq.new_empty((4, Cout)), bits, x_amax,
            *_fake_running(x_seq, batch_stats, running_mean, running_var))


@torch.library.custom_op("sj::hip_conv_bn_lif_backward", mutates_args=())
def hip_conv_bn_lif_backward(grad_out: Optional[torch.Tensor], grad_v_last: Optional[torch.Tensor], x_seq: torch.Tensor,
                             weight: torch.Tensor, gamma: Optional[torch.Tensor], v_init: torch.Tensor, y: torch.Tensor,
                             bn_map: torch.Tensor, bits: torch.Tensor, x_amax: torch.Tensor, batch_stats: bool, tau: float,
                             v_th: float, v_reset: float, flags: int, sg_id: int, sg_alpha: float, x_exact: bool, terms: int,
                             heads: int, cph: int, scale: float, need_dx: bool, need_dw: bool, need_gvi: bool,
                             k: Optional[torch.Tensor] = None
                             ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    if terms != C._terms():
        raise RuntimeError("configure.hip_conv_split / hip_conv_terms changed after this call was compiled")
    spec = (tau, v_th, v_reset, flags, sg_id, sg_alpha)
    ssa = (heads, cph, scale) if heads else None
    dx, dw, dgamma, dbeta, gvi, *grad_k = C._conv_chain_backward(L.aligned16(x_seq), weight, gamma, v_init, y, bn_map, bits, x_amax,
                                                                 spec, batch_stats, x_exact, ssa, grad_out, grad_v_last, need_dx,
                                                                 need_dw, need_gvi, k)
    return (_or_empty(dx, y), _or_empty(dw, y), dgamma.clone(), dbeta.clone(), _or_empty(gvi, y),
            grad_k[0] if grad_k else _e(y))


@hip_conv_bn_lif_backward.register_fake
def _(grad_out, grad_v_last, x_seq, weight, gamma, v_init, y, bn_map, bits, x_amax, batch_stats, tau, v_th, v_reset, flags,
      sg_id, sg_alpha, x_exact, terms, heads, cph, scale, need_dx, need_dw, need_gvi, k=None):
    T, B, Cout, Lp = y.shape
    return (torch.empty_like(x_seq) if need_dx else _e(y), y.new_empty(tuple(weight.shape[:2])) if need_dw else _e(y),
            y.new_empty((Cout,)), y.new_empty((Cout,)), y.new_empty((B, Cout, Lp) if need_gvi else (0,)),
            y.new_empty((1,) if k is not None else (0,)))


def _conv_setup(ctx, inputs, output):
    (x_seq, weight, gamma, beta, v_init, running_mean, running_var, batch_stats, momentum, eps, tau, v_th, v_reset,
     flags, sg_id, sg_alpha, x_exact, terms, heads, cph, scale, k) = inputs
    ctx.scalars = (batch_stats, tau, v_th, v_reset, flags, sg_id, sg_alpha, x_exact, terms, heads, cph, scale)
    ctx.save_for_backward(x_seq, weight, gamma, v_init, output[2], output[3], output[4], output[5], k)
    ctx.set_materialize_grads(False)


def _conv_formula(ctx, grad_out, grad_v_last, _y, _map, _bits, _amax, _rm, _rv):
    x_seq, weight, gamma, v_init, y, bn_map, bits, x_amax, k = ctx.saved_tensors
    need = ctx.needs_input_grad
    dx, dw, dgamma, dbeta, gvi, grad_k = hip_conv_bn_lif_backward(grad_out, grad_v_last, x_seq, weight, gamma, v_init, y, bn_map,
                                                                  bits, x_amax, *ctx.scalars, bool(need[0]), bool(need[1]),
                                                                  bool(need[4]), k)
    dw = dw.view(weight.shape) if need[1] else None
    return (dx if need[0] else None, dw, dgamma if need[2] else None, dbeta if need[3] else None,
            gvi if need[4] else None) + (None,) * 16 + (grad_k if k is not None and need[21] else None,)


torch.library.register_autograd("sj::hip_conv_bn_lif_forward", _conv_formula, setup_context=_conv_setup)


def conv_bn_lif(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact: bool, ssa, k=None):
    """``(spikes, v_last)``, or with ``ssa = (heads, channels per head, scale)`` ``(contraction output, v_last)``."""
    running_mean, running_var, batch_stats, momentum, eps, _ = C._bn_config(bn)
    heads, cph, scale = ssa if ssa is not None else (0, 0, 0.0)
    out = hip_conv_bn_lif_forward(x_seq, weight, gamma, beta, v_init, running_mean, running_var, batch_stats, momentum,
                                  eps, *spec, x_exact, C._terms(), heads, cph, scale, k)
    _write_back(bn, out[6], out[7])
    return out[0], out[1]


# =================================================================================================
# LIF (bits) + convolution + batch norm + LIF
# =================================================================================================
@torch.library.custom_op("sj::hip_lif_conv_bn_lif_forward", mutates_args=())
def hip_lif_conv_bn_lif_forward(pre_seq: torch.Tensor, pre_v_init: torch.Tensor, weight: torch.Tensor,
                                gamma: Optional[torch.Tensor], beta: Optional[torch.Tensor], v_init: torch.Tensor,
                                running_mean: Optional[torch.Tensor], running_var: Optional[torch.Tensor],
                                batch_stats: bool, momentum: float, eps: float,
                                pre_tau: float, pre_v_th: float, pre_v_reset: float, pre_flags: int, pre_sg_id: int,
                                pre_sg_alpha: float, tau: float, v_th: float, v_reset: float, flags: int, sg_id: int,
                                sg_alpha: float, terms: int, k: Optional[torch.Tensor] = None
                                ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                                           torch.Tensor, torch.Tensor]:
    """``(spikes, v_last, first neuron's v_last, y, bn_map, bits, new running mean, new running variance)``."""
    if terms != C._terms():
        raise RuntimeError("configure.hip_conv_split / hip_conv_terms changed after this call was compiled")
    rm, rv, upd = _updated(batch_stats, running_mean, running_var)
    out = C._LifConvBnLif.forward(pre_seq, pre_v_init, weight, gamma, beta, v_init,
                                  (rm, rv, batch_stats, momentum, eps, None),
                                  (pre_tau, pre_v_th, pre_v_reset, pre_flags, pre_sg_id, pre_sg_alpha),
                                  (tau, v_th, v_reset, flags, sg_id, sg_alpha), k)
    return (*out, rm if upd else _e(pre_seq), rv if upd else _e(pre_seq))


@hip_lif_conv_bn_lif_forward.register_fake
def _(pre_seq, pre_v_init, weight, gamma, beta, v_init, running_mean, running_var, batch_stats, momentum, eps, pre_tau,
      pre_v_th, pre_v_reset, pre_flags, pre_sg_id, pre_sg_alpha, tau, v_th, v_reset, flags, sg_id, sg_alpha, terms, k=None):
    T, B, Cin, Lp = pre_seq.shape
    Cout = weight.shape[0]
    new = pre_seq.new_empty
    return (new((T, B, Cout, Lp)), new((B, Cout, Lp)), new((B, Cin, Lp)), new((T, B, Cout, Lp)), new((4, Cout)),
            torch.empty((T * B * Cin * Lp // 8,), dtype=torch.uint8, device=pre_seq.device),
            *_fake_running(pre_seq, batch_stats, running_mean, running_var))


@torch.library.custom_op("sj::hip_lif_conv_bn_lif_backward", mutates_args=())
def hip_lif_conv_bn_lif_backward(grad_spikes: Optional[torch.Tensor], grad_v_last: Optional[torch.Tensor],
                                 grad_pre_v_last: Optional[torch.Tensor], pre_seq: torch.Tensor, pre_v_init: torch.Tensor,
                                 weight: torch.Tensor, gamma: Optional[torch.Tensor], v_init: torch.Tensor, y: torch.Tensor,
                                 bn_map: torch.Tensor, bits: torch.Tensor, batch_stats: bool, pre_tau: float, pre_v_th: float,
                                 pre_v_reset: float, pre_flags: int, pre_sg_id: int, pre_sg_alpha: float, tau: float,
                                 v_th: float, v_reset: float, flags: int, sg_id: int, sg_alpha: float, terms: int,
                                 need_gx: bool, need_gpv: bool, need_dw: bool, need_gvi: bool, k: Optional[torch.Tensor] = None
                                 ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                                            torch.Tensor]:
    if terms != C._terms():
        raise RuntimeError("configure.hip_conv_split / hip_conv_terms changed after this call was compiled")
    gx, gpv, dw, dgamma, dbeta, gvi, *grad_k = C._lif_conv_chain_backward(
        L.aligned16(pre_seq), pre_v_init, weight, gamma, v_init, y, bn_map, bits,
        (pre_tau, pre_v_th, pre_v_reset, pre_flags, pre_sg_id, pre_sg_alpha), (tau, v_th, v_reset, flags, sg_id, sg_alpha),
        batch_stats, grad_spikes, grad_v_last, grad_pre_v_last, need_gx, need_gpv, need_dw, need_gvi, k)
    return (_or_empty(gx, y), _or_empty(gpv, y), _or_empty(dw, y), dgamma.clone(), dbeta.clone(), _or_empty(gvi, y),
            grad_k[0] if grad_k else _e(y))


@hip_lif_conv_bn_lif_backward.register_fake
def _(grad_spikes, grad_v_last, grad_pre_v_last, pre_seq, pre_v_init, weight, gamma, v_init, y, bn_map, bits, batch_stats,
      pre_tau, pre_v_th, pre_v_reset, pre_flags, pre_sg_id, pre_sg_alpha, tau, v_th, v_reset, flags, sg_id, sg_alpha, terms,
      need_gx, need_gpv, need_dw, need_gvi, k=None):
    T, B, Cin, Lp = pre_seq.shape
    Cout = weight.shape[0]
    new = y.new_empty
    return (torch.empty_like(pre_seq) if need_gx else _e(y), new((B, Cin, Lp)) if need_gpv else _e(y),
            new((Cout, Cin)) if need_dw else _e(y), new((Cout,)), new((Cout,)), new((B, Cout, Lp)) if need_gvi else _e(y),
            new((1,) if k is not None else (0,)))


def _lif_conv_setup(ctx, inputs, output):
    (pre_seq, pre_v_init, weight, gamma, beta, v_init, running_mean, running_var, batch_stats, momentum, eps,
     *scalars, k) = inputs
    ctx.scalars = (batch_stats, *scalars)
    ctx.save_for_backward(pre_seq, pre_v_init, weight, gamma, v_init, output[3], output[4], output[5], k)
    ctx.set_materialize_grads(False)


def _lif_conv_formula(ctx, grad_spikes, grad_v_last, grad_pre_v_last, _y, _map, _bits, _rm, _rv):
    pre_seq, pre_v_init, weight, gamma, v_init, y, bn_map, bits, k = ctx.saved_tensors
    need = ctx.needs_input_grad
    gx, gpv, dw, dgamma, dbeta, gvi, grad_k = hip_lif_conv_bn_lif_backward(
        grad_spikes, grad_v_last, grad_pre_v_last, pre_seq, pre_v_init, weight, gamma, v_init, y, bn_map, bits, *ctx.scalars,
        bool(need[0]), bool(need[1]), bool(need[2]), bool(need[5]), k)
    dw = dw.view(weight.shape) if need[2] else None
    return (gx if need[0] else None, gpv if need[1] else None, dw, dgamma if need[3] else None, dbeta if need[4] else None,
            gvi if need[5] else None) + (None,) * 18 + (grad_k if k is not None and need[24] else None,)


torch.library.register_autograd("sj::hip_lif_conv_bn_lif_forward", _lif_conv_formula, setup_context=_lif_conv_setup)


def lif_conv_bn_lif(pre_seq, pre_v_init, weight, gamma, beta, v_init, bn, pre_spec, spec, k=None):
    running_mean, running_var, batch_stats, momentum, eps, _ = C._bn_config(bn)
    out = hip_lif_conv_bn_lif_forward(pre_seq, pre_v_init, weight, gamma, beta, v_init, running_mean, running_var,
                                      batch_stats, momentum, eps, *pre_spec, *spec, C._terms(), k)
    _write_back(bn, out[6], out[7])
    return out[0], out[1], out[2]


# =================================================================================================
# LIF (bits) + contraction
# =================================================================================================
@torch.library.custom_op("sj::hip_lif_ssa_forward", mutates_args=())
def hip_lif_ssa_forward(x_seq: torch.Tensor, v_init: torch.Tensor, tau: float, v_th: float, v_reset: float, flags: int,
                        sg_id: int, sg_alpha: float, samples: int, heads: int, cph: int, tokens: int, scale: float
                        ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(out [samples, heads, cph, tokens], v_last, bits)`` for ``x_seq [T, N]``."""
    return A._LifSsa.forward(x_seq, v_init, (tau, v_th, v_reset, flags, sg_id, sg_alpha, samples, heads, cph, tokens, scale))


@hip_lif_ssa_forward.register_fake
def _(x_seq, v_init, tau, v_th, v_reset, flags, sg_id, sg_alpha, samples, heads, cph, tokens, scale):
    return (x_seq.new_empty((samples, heads, cph, tokens)), x_seq.new_empty((x_seq.shape[1],)),
            torch.empty((x_seq.numel() // 8,), dtype=torch.uint8, device=x_seq.device))


@torch.library.custom_op("sj::hip_lif_ssa_backward", mutates_args=())
def hip_lif_ssa_backward(grad_out: Optional[torch.Tensor], grad_v_last: Optional[torch.Tensor], x_seq: torch.Tensor,
                         v_init: torch.Tensor, bits: torch.Tensor, tau: float, v_th: float, v_reset: float, flags: int,
                         sg_id: int, sg_alpha: float, samples: int, heads: int, cph: int, tokens: int, scale: float,
                         need_gvi: bool) -> tuple[torch.Tensor, torch.Tensor]:
    gx, gvi = A._lif_ssa_backward(x_seq, v_init, bits, (tau, v_th, v_reset, flags, sg_id, sg_alpha, samples, heads, cph, tokens,
                                                       scale), grad_out, grad_v_last, need_gvi)
    return gx, _or_empty(gvi, x_seq)


@hip_lif_ssa_backward.register_fake
def _(grad_out, grad_v_last, x_seq, v_init, bits, tau, v_th, v_reset, flags, sg_id, sg_alpha, samples, heads, cph, tokens, scale,
      need_gvi):
    return torch.empty_like(x_seq), x_seq.new_empty((x_seq.shape[1],) if need_gvi else (0,))


def _lif_ssa_setup(ctx, inputs, output):
    x_seq, v_init, *scalars = inputs
    ctx.scalars = tuple(scalars)
    ctx.save_for_backward(x_seq, v_init, output[2])
    ctx.set_materialize_grads(False)


def _lif_ssa_formula(ctx, grad_out, grad_v_last, _bits):
    x_seq, v_init, bits = ctx.saved_tensors
    need = bool(ctx.needs_input_grad[1])
    gx, gvi = hip_lif_ssa_backward(grad_out, grad_v_last, x_seq, v_init, bits, *ctx.scalars, need)
    return (gx, gvi if need else None) + (None,) * 11


torch.library.register_autograd("sj::hip_lif_ssa_forward", _lif_ssa_formula, setup_context=_lif_ssa_setup)


def lif_ssa(x_seq, v_init, spec):
    out, v_last, _ = hip_lif_ssa_forward(x_seq, v_init, *spec)
    return out, v_last
