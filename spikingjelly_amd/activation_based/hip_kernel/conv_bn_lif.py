"""Kernel-size-1 convolution, batch normalisation and the multi-step LIF that follows them, on the hip kernels.

The block ``SeqToANNContainer(Conv1d(k=1, bias=False), BatchNorm1d) -> LIFNode`` appears twice in the reference's
``SpikingSelfAttention`` (layer/attention.py:310-329, 370-384) and, with ``Conv2d`` / ``BatchNorm2d``, in
``SpikformerConv2dBNLIF`` (model/spikformer.py:107-212); there torch runs the convolution (MIOpen / hipBLASLt, with
layout transposes around them), batch norm and the neuron as separate operators.  Here, for fp32 ``[T, B, C, L]``
tensors (``L`` the flattened positions, a multiple of 4):

* the convolution and its two gradients are GEMMs on the bf16 matrix cores with the fp32 operands split into up to
  three bf16 terms (``csrc/pwconv.hip``; ``configure.hip_conv_terms`` = 3 keeps fp32 accuracy, 2 and 1 trade it for speed;
  an input that is known to be spikes needs one term);
* batch norm and the neuron are two passes over the convolution output (``csrc/bn_lif.hip``): per-channel statistics,
  then normalise + charge + fire + reset over the T steps in registers, spikes written dense or bit-packed; the
  normalised tensor never exists.  The backward replays the neuron from the convolution output.

Three entries share the pieces: ``bn_lif`` (any convolution output, e.g. a 3x3 ``Conv2d`` run by torch),
``conv_bn_lif`` (the whole block) and ``conv_bn_lif_ssa`` (the block feeding the spiking self-attention contraction
through bit-packed spikes).  All are ``autograd.Function`` s around plain launch helpers; nothing here falls back to
another implementation: callers check ``supported()`` first and keep torch's operators for what it refuses.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ... import configure
from . import library as L
from . import neuron_kernel as K

__all__ = ["supported", "bn_lif", "conv_bn_lif", "conv_bn_lif_ssa", "conv_bn_lif_ssa_lif", "split_weight", "pw_gemm",
           "pw_grad_weight"]

MAX_REPLAY_STEPS = 16  # the backward replays the neuron with h of every step in registers


def _terms() -> int:
    t = int(getattr(configure, "hip_conv_terms", 3))
    if t not in (1, 2, 3):
        raise ValueError(f"configure.hip_conv_terms must be 1, 2 or 3, got {t}")
    return t


def supported(x_seq: torch.Tensor, need_grad: bool) -> bool:
    """fp32 device tensor ``[T, B, C, L]`` whose rows of ``L`` elements start on 16 bytes; at most 16 steps when a
    backward will follow."""
    return (x_seq.is_cuda and x_seq.dtype == torch.float32 and x_seq.dim() == 4 and x_seq.shape[-1] % 4 == 0
            and x_seq.numel() > 0 and (not need_grad or x_seq.shape[0] <= MAX_REPLAY_STEPS))


def _stream(t: torch.Tensor) -> int:
    return L.current_stream_ptr(t.device)


# ------------------------------------------------------------------------------------------------
# launch helpers (no autograd)
# ------------------------------------------------------------------------------------------------
def split_weight(weight: torch.Tensor, transpose: bool) -> torch.Tensor:
    """bf16 term planes ``[3, rows_pad, cols_pad]`` of ``weight [Cout, Cin]`` (or of its transpose): the A operand of
    ``pw_gemm``."""
    rows, cols = weight.shape
    w = L.aligned16(weight.detach().to(torch.float32))
    planes = torch.empty(L.load().sjhip_pwconv_planes_elems(cols if transpose else rows, rows if transpose else cols),
                         dtype=torch.bfloat16, device=weight.device)
    with torch.cuda.device(weight.device):
        rc = L.load().sjhip_pwconv_split_weight(w.data_ptr(), rows, cols, 1 if transpose else 0, planes.data_ptr(), _stream(w))
    L.check(rc, "pwconv_split_weight")
    return planes


def pw_gemm(planes: torch.Tensor, a_terms: int, M: int, Kdim: int, b: torch.Tensor, b_terms: int, stats: bool = False):
    """``c[s] = A b[s]`` for ``b [S, K, L]`` -> ``c [S, M, L]``.  With ``stats`` the result is ``(c, partial)``:
    ``partial [rows, M, 2]`` holds sums and sums of squares of every row of ``c`` over groups of its columns, the input
    of ``_bn_map``."""
    S, Kb, Lp = b.shape
    assert Kb == Kdim
    b = L.aligned16(b)
    c = torch.empty((S, M, Lp), dtype=torch.float32, device=b.device)
    lib = L.load()
    with torch.cuda.device(b.device):
        if stats:
            rows = lib.sjhip_pwconv_gemm_stats_rows(Kdim, S, Lp)
            partial = torch.empty((rows, M, 2), dtype=torch.float32, device=b.device)
            rc = lib.sjhip_pwconv_gemm_stats(planes.data_ptr(), a_terms, M, Kdim, b.data_ptr(), b_terms, S, Lp, c.data_ptr(),
                                             partial.data_ptr(), _stream(b))
        else:
            rc = lib.sjhip_pwconv_gemm(planes.data_ptr(), a_terms, M, Kdim, b.data_ptr(), b_terms, S, Lp, c.data_ptr(), _stream(b))
    L.check(rc, "pwconv_gemm")
    return (c, partial) if stats else c


def pw_grad_weight(dy: torch.Tensor, dy_terms: int, x: torch.Tensor, x_terms: int) -> torch.Tensor:
    """``dw[m, n] = sum_{s, l} dy[s, m, l] x[s, n, l]``."""
    S, M, Lp = dy.shape
    N = x.shape[1]
    dy, x = L.aligned16(dy), L.aligned16(x)
    lib = L.load()
    ws = torch.empty(lib.sjhip_pwconv_grad_weight_workspace_floats(M, N, S), dtype=torch.float32, device=dy.device)
    dw = torch.empty((M, N), dtype=torch.float32, device=dy.device)
    with torch.cuda.device(dy.device):
        rc = lib.sjhip_pwconv_grad_weight(dy.data_ptr(), dy_terms, x.data_ptr(), x_terms, S, M, N, Lp, dw.data_ptr(),
                                          ws.data_ptr(), _stream(dy))
    L.check(rc, "pwconv_grad_weight")
    return dw


def _bn_map(y: torch.Tensor, gamma, beta, running_mean, running_var, batch_stats: bool, momentum: float, eps: float,
            partial: Optional[torch.Tensor] = None):
    """Per-channel ``(scale, shift, mean, invstd)`` of ``z = y * scale + shift`` for ``y [S, C, L]``; with
    ``batch_stats`` from the statistics of ``y`` (and the running statistics, when given, are updated in place).
    ``partial``: the sums the convolution left behind (``pw_gemm(..., stats=True)``), which save the pass over ``y``."""
    S, C, Lp = y.shape
    lib = L.load()
    out = torch.empty((4, C), dtype=torch.float32, device=y.device)
    with torch.cuda.device(y.device):
        if batch_stats and partial is not None:
            rc = lib.sjhip_bn_finalize_rows(partial.data_ptr(), partial.shape[0], S * Lp, C, L.ptr(gamma), L.ptr(beta), eps,
                                            momentum, L.ptr(running_mean), L.ptr(running_var), out[0].data_ptr(),
                                            out[1].data_ptr(), out[2].data_ptr(), out[3].data_ptr(), _stream(y))
            L.check(rc, "bn_finalize_rows")
            return out
        partial = None
        if batch_stats:
            partial = torch.empty((S * C, 2), dtype=torch.float32, device=y.device)
            L.check(lib.sjhip_bn_stats(y.data_ptr(), S, C, Lp, partial.data_ptr(), _stream(y)), "bn_stats")
        rc = lib.sjhip_bn_finalize(L.ptr(partial), S, C, Lp, L.ptr(gamma), L.ptr(beta), eps, momentum, L.ptr(running_mean),
                                   L.ptr(running_var), out[0].data_ptr(), out[1].data_ptr(), out[2].data_ptr(),
                                   out[3].data_ptr(), _stream(y))
    L.check(rc, "bn_finalize")
    return out


def _lif_params(spec, flags_extra: int = 0) -> L.NeuronParams:
    tau, v_th, v_reset, flags, sg_id, sg_alpha = spec
    return K._params(tau, v_th, v_reset, sg_alpha, sg_id, flags | flags_extra)


def _bn_lif_forward(y: torch.Tensor, bn_map: torch.Tensor, v_init: torch.Tensor, spec, packed: bool):
    """``y [T, B, C, L]`` -> (spikes ``[T, B, C, L]`` fp32 or the bit-packed byte array, ``v_last [B, C, L]``)."""
    T, B, C, Lp = y.shape
    v_keep, broadcast = K._state_arg(v_init, True)
    params = _lif_params(spec, broadcast)
    v_last = torch.empty((B, C, Lp), dtype=torch.float32, device=y.device)
    if packed:
        spikes = torch.empty((T * B * C * Lp // 8,), dtype=torch.uint8, device=y.device)
    else:
        spikes = torch.empty_like(y)
    with torch.cuda.device(y.device):
        rc = L.load().sjhip_bn_lif_forward(L.NEURON_LIF, ctypes.byref(params), T, B, C, Lp, y.data_ptr(), bn_map[0].data_ptr(),
                                           bn_map[1].data_ptr(), v_keep.data_ptr(), None if packed else spikes.data_ptr(),
                                           spikes.data_ptr() if packed else None, v_last.data_ptr(), _stream(y))
    L.check(rc, "bn_lif_forward")
    return spikes, v_last


def _bn_lif_backward(y: torch.Tensor, bn_map: torch.Tensor, gamma, v_init: torch.Tensor, spec, batch_stats: bool,
                     grad_spikes: Optional[torch.Tensor], grad_v_last: Optional[torch.Tensor], need_grad_v_init: bool):
    """Returns ``(dy [T, B, C, L], dgamma [C], dbeta [C], grad_v_init or None)``."""
    T, B, C, Lp = y.shape
    lib = L.load()
    if grad_spikes is None:
        grad_spikes = torch.zeros_like(y)
    grad_spikes = L.aligned16(grad_spikes.to(torch.float32))
    if grad_v_last is not None:
        grad_v_last = L.aligned16(grad_v_last.to(torch.float32))
    v_keep, broadcast = K._state_arg(v_init, True)
    params = _lif_params(spec, broadcast)
    g = torch.empty_like(y)
    partial = torch.empty((B * C, 2), dtype=torch.float32, device=y.device)
    grads = torch.empty((5, C), dtype=torch.float32, device=y.device)  # dgamma, dbeta, then the coefficients p, q, r
    grad_v_init = torch.empty((B, C, Lp), dtype=torch.float32, device=y.device) if need_grad_v_init else None
    with torch.cuda.device(y.device):
        stream = _stream(y)
        L.check(lib.sjhip_bn_lif_backward(L.NEURON_LIF, ctypes.byref(params), T, B, C, Lp, y.data_ptr(), bn_map[0].data_ptr(),
                                          bn_map[1].data_ptr(), v_keep.data_ptr(), grad_spikes.data_ptr(), L.ptr(grad_v_last),
                                          g.data_ptr(), L.ptr(grad_v_init), partial.data_ptr(), stream), "bn_lif_backward")
        L.check(lib.sjhip_bn_backward_finalize(partial.data_ptr(), T, B, C, Lp, 1 if batch_stats else 0, L.ptr(gamma),
                                               bn_map[2].data_ptr(), bn_map[3].data_ptr(), grads[0].data_ptr(),
                                               grads[1].data_ptr(), grads[2].data_ptr(), stream), "bn_backward_finalize")
        L.check(lib.sjhip_bn_grad_input(g.data_ptr(), y.data_ptr(), grads[2].data_ptr(), T * B, C, Lp, g.data_ptr(), stream),
                "bn_grad_input")
    return g, grads[0], grads[1], grad_v_init


# ------------------------------------------------------------------------------------------------
# autograd
# ------------------------------------------------------------------------------------------------
# bn: (running_mean | None, running_var | None, batch_stats, momentum, eps)
# lif spec: (tau, v_threshold, v_reset, flags, sg_id, sg_alpha)
def _conv_forward(x_seq, weight, x_exact, stats: bool = False):
    """``y [T, B, Cout, L]``, and with ``stats`` the partial batch-norm sums of ``y`` as well."""
    T, B, Cin, Lp = x_seq.shape
    Cout = weight.shape[0]
    terms = _terms()
    planes = split_weight(weight, False)
    out = pw_gemm(planes, terms, Cout, Cin, x_seq.reshape(T * B, Cin, Lp), 1 if x_exact else terms, stats)
    if stats:
        return out[0].view(T, B, Cout, Lp), out[1]
    return out.view(T, B, Cout, Lp)


def _conv_backward(dy, x_seq, weight, x_exact, need_dx, need_dw):
    T, B, Cin, Lp = x_seq.shape
    Cout = weight.shape[0]
    terms = _terms()
    dy3 = dy.view(T * B, Cout, Lp)
    dw = pw_grad_weight(dy3, terms, x_seq.reshape(T * B, Cin, Lp), 1 if x_exact else terms) if need_dw else None
    dx = None
    if need_dx:
        dx = pw_gemm(split_weight(weight, True), terms, Cin, Cout, dy3, terms).view(T, B, Cin, Lp)
    return dx, dw


class _BnLif(torch.autograd.Function):
    @staticmethod
    def forward(y, gamma, beta, v_init, bn, spec):
        running_mean, running_var, batch_stats, momentum, eps = bn
        y = L.aligned16(y)
        bn_map = _bn_map(y.flatten(0, 1), gamma, beta, running_mean, running_var, batch_stats, momentum, eps)
        spikes, v_last = _bn_lif_forward(y, bn_map, v_init, spec, False)
        return spikes, v_last, bn_map

    @staticmethod
    def setup_context(ctx, inputs, output):
        y, gamma, beta, v_init, bn, spec = inputs
        ctx.spec, ctx.batch_stats = spec, bn[2]
        ctx.save_for_backward(L.aligned16(y), gamma, v_init, output[2])
        ctx.mark_non_differentiable(output[2])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_spikes, grad_v_last, _):
        y, gamma, v_init, bn_map = ctx.saved_tensors
        need = ctx.needs_input_grad
        dy, dgamma, dbeta, gvi = _bn_lif_backward(y, bn_map, gamma, v_init, ctx.spec, ctx.batch_stats, grad_spikes,
                                                  grad_v_last, bool(need[3]))
        return (dy if need[0] else None, dgamma if need[1] else None, dbeta if need[2] else None, gvi, None, None)


class _ConvBnLif(torch.autograd.Function):
    @staticmethod
    def forward(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact):
        running_mean, running_var, batch_stats, momentum, eps = bn
        x_seq = L.aligned16(x_seq)
        y, partial = _conv_forward(x_seq, weight, x_exact, True) if batch_stats else (_conv_forward(x_seq, weight, x_exact), None)
        bn_map = _bn_map(y.flatten(0, 1), gamma, beta, running_mean, running_var, batch_stats, momentum, eps, partial)
        spikes, v_last = _bn_lif_forward(y, bn_map, v_init, spec, False)
        return spikes, v_last, y, bn_map

    @staticmethod
    def setup_context(ctx, inputs, output):
        x_seq, weight, gamma, beta, v_init, bn, spec, x_exact = inputs
        ctx.spec, ctx.batch_stats, ctx.x_exact = spec, bn[2], x_exact
        ctx.save_for_backward(L.aligned16(x_seq), weight, gamma, v_init, output[2], output[3])
        ctx.mark_non_differentiable(output[2], output[3])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_spikes, grad_v_last, _y, _map):
        x_seq, weight, gamma, v_init, y, bn_map = ctx.saved_tensors
        need = ctx.needs_input_grad
        dy, dgamma, dbeta, gvi = _bn_lif_backward(y, bn_map, gamma, v_init, ctx.spec, ctx.batch_stats, grad_spikes,
                                                  grad_v_last, bool(need[4]))
        dx, dw = _conv_backward(dy, x_seq, weight, ctx.x_exact, bool(need[0]), bool(need[1]))
        return (dx, dw, dgamma if need[2] else None, dbeta if need[3] else None, gvi, None, None, None)


class _ConvBnLifSsa(torch.autograd.Function):
    """The qkv half of the spiking self-attention: convolution, batch norm, LIF with bit-packed spike output, and the
    contraction ``scale (V K^T) Q`` reading those bits.  Saves the input, the convolution output and the bits."""

    @staticmethod
    def forward(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, ssa):
        from . import attention_kernel as A

        running_mean, running_var, batch_stats, momentum, eps = bn
        heads, cph, scale = ssa
        x_seq = L.aligned16(x_seq)
        T, B, _, Lp = x_seq.shape
        y, partial = _conv_forward(x_seq, weight, x_exact, True) if batch_stats else (_conv_forward(x_seq, weight, x_exact), None)
        bn_map = _bn_map(y.flatten(0, 1), gamma, beta, running_mean, running_var, batch_stats, momentum, eps, partial)
        bits, v_last = _bn_lif_forward(y, bn_map, v_init, spec, True)
        out = A._ssa_packed(bits, None, torch.float32, T * B, heads, cph, Lp, scale)
        return out, v_last, y, bn_map, bits

    @staticmethod
    def setup_context(ctx, inputs, output):
        x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, ssa = inputs
        ctx.spec, ctx.batch_stats, ctx.x_exact, ctx.ssa = spec, bn[2], x_exact, ssa
        ctx.save_for_backward(L.aligned16(x_seq), weight, gamma, v_init, output[2], output[3], output[4])
        ctx.mark_non_differentiable(output[2], output[3], output[4])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_out, grad_v_last, _y, _map, _bits):
        from . import attention_kernel as A

        x_seq, weight, gamma, v_init, y, bn_map, bits = ctx.saved_tensors
        heads, cph, scale = ctx.ssa
        T, B, _, Lp = x_seq.shape
        need = ctx.needs_input_grad
        grad_spikes = None
        if grad_out is not None:
            grad_spikes = A._ssa_packed(bits, grad_out, torch.float32, T * B, heads, cph, Lp, scale).view(y.shape)
        dy, dgamma, dbeta, gvi = _bn_lif_backward(y, bn_map, gamma, v_init, ctx.spec, ctx.batch_stats, grad_spikes,
                                                  grad_v_last, bool(need[4]))
        dx, dw = _conv_backward(dy, x_seq, weight, ctx.x_exact, bool(need[0]), bool(need[1]))
        return (dx, dw, dgamma if need[2] else None, dbeta if need[3] else None, gvi, None, None, None, None)


class _ConvBnLifSsaLif(torch.autograd.Function):
    """``_ConvBnLifSsa`` followed by the attention's own LIF, whose input ``scale (V K^T) Q`` never leaves the kernel
    that computes it.  Saves the input, the convolution output, the bits and, when a gradient is wanted, the attention
    neuron's ``h_seq``."""

    @staticmethod
    def forward(x_seq, weight, gamma, beta, v_init, attn_v_init, bn, spec, x_exact, ssa, attn_spec, save_h):
        from . import attention_kernel as A

        running_mean, running_var, batch_stats, momentum, eps = bn
        heads, cph, scale = ssa
        x_seq = L.aligned16(x_seq)
        T, B, _, Lp = x_seq.shape
        y, partial = _conv_forward(x_seq, weight, x_exact, True) if batch_stats else (_conv_forward(x_seq, weight, x_exact), None)
        bn_map = _bn_map(y.flatten(0, 1), gamma, beta, running_mean, running_var, batch_stats, momentum, eps, partial)
        bits, v_last = _bn_lif_forward(y, bn_map, v_init, spec, True)
        v_keep, broadcast = K._state_arg(attn_v_init, True)
        spikes, h_seq, attn_v_last = A._ssa_lif_forward(bits, v_keep, _lif_params(attn_spec, broadcast), T, B, heads, cph,
                                                        Lp, scale, save_h)
        if h_seq is None:
            h_seq = spikes.new_empty((0,))
        return spikes, v_last, attn_v_last, y, bn_map, bits, h_seq

    @staticmethod
    def setup_context(ctx, inputs, output):
        x_seq, weight, gamma, beta, v_init, attn_v_init, bn, spec, x_exact, ssa, attn_spec, save_h = inputs
        ctx.spec, ctx.batch_stats, ctx.x_exact, ctx.ssa, ctx.attn_spec = spec, bn[2], x_exact, ssa, attn_spec
        ctx.save_for_backward(L.aligned16(x_seq), weight, gamma, v_init, output[3], output[4], output[5], output[6])
        ctx.mark_non_differentiable(output[3], output[4], output[5], output[6])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_attn_spikes, grad_v_last, grad_attn_v_last, _y, _map, _bits, _h):
        from . import attention_kernel as A

        x_seq, weight, gamma, v_init, y, bn_map, bits, h_seq = ctx.saved_tensors
        if h_seq.numel() == 0:
            raise RuntimeError("the fused attention block was run without saving h_seq and cannot be differentiated")
        heads, cph, scale = ctx.ssa
        T, B, _, Lp = x_seq.shape
        need = ctx.needs_input_grad
        grad_spikes = None
        if grad_attn_spikes is not None or grad_attn_v_last is not None:
            grad_qkv, _ = A._ssa_lif_backward(bits, h_seq, grad_attn_spikes, grad_attn_v_last, _lif_params(ctx.attn_spec), T, B,
                                              heads, cph, Lp, scale, False)
            grad_spikes = grad_qkv.view(y.shape)
        dy, dgamma, dbeta, gvi = _bn_lif_backward(y, bn_map, gamma, v_init, ctx.spec, ctx.batch_stats, grad_spikes,
                                                  grad_v_last, bool(need[4]))
        dx, dw = _conv_backward(dy, x_seq, weight, ctx.x_exact, bool(need[0]), bool(need[1]))
        return (dx, dw, dgamma if need[2] else None, dbeta if need[3] else None, gvi, None, None, None, None, None, None, None)


def bn_lif(y_seq: torch.Tensor, gamma, beta, v_init: torch.Tensor, bn, spec):
    """``y_seq [T, B, C, L]`` (a convolution output) -> ``(spikes, v_last)``."""
    spikes, v_last, _ = _BnLif.apply(y_seq, gamma, beta, v_init, bn, spec)
    return spikes, v_last


def conv_bn_lif(x_seq: torch.Tensor, weight: torch.Tensor, gamma, beta, v_init: torch.Tensor, bn, spec, x_exact: bool):
    """``x_seq [T, B, Cin, L]``, ``weight [Cout, Cin]`` -> ``(spikes [T, B, Cout, L], v_last [B, Cout, L])``.
    ``x_exact``: every element of ``x_seq`` is exactly representable in bf16 (spikes, small integers)."""
    spikes, v_last, _, _ = _ConvBnLif.apply(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact)
    return spikes, v_last


def conv_bn_lif_ssa(x_seq: torch.Tensor, weight: torch.Tensor, gamma, beta, v_init: torch.Tensor, bn, spec, x_exact: bool,
                    heads: int, channels_per_head: int, scale: float):
    """The same block with ``Cout = 3 * heads * channels_per_head`` followed by the contraction; returns
    ``(out [T * B, heads, channels_per_head, L], v_last)``."""
    out, v_last, _, _, _ = _ConvBnLifSsa.apply(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact,
                                               (heads, channels_per_head, scale))
    return out, v_last


def conv_bn_lif_ssa_lif(x_seq: torch.Tensor, weight: torch.Tensor, gamma, beta, v_init: torch.Tensor, attn_v_init: torch.Tensor,
                        bn, spec, x_exact: bool, heads: int, channels_per_head: int, scale: float, attn_spec, save_h: bool):
    """``conv_bn_lif_ssa`` followed by the LIF of ``attn_spec`` on the contraction's output; returns
    ``(spikes [T, B, heads, channels_per_head, L], v_last of the first neuron, v_last of the attention neuron)``."""
    out = _ConvBnLifSsaLif.apply(x_seq, weight, gamma, beta, v_init, attn_v_init, bn, spec, x_exact,
                                 (heads, channels_per_head, scale), attn_spec, save_h)
    return out[0], out[1], out[2]
