"""``torch.library`` operators for the multi-step IF / LIF / PLIF kernels of ``libsjhip.so``.

Operator layout follows the reference's kernel backends
(``cuda_kernel/neuron_kernel/multi_step/lif.py:144-325``: forward op + fake + backward op +
``register_autograd`` saving ``h_seq``; ``triton_kernel/neuron_kernel/lif.py:673-763``: a separate
inference op that writes no ``h_seq``):

    sj::hip_multistep_{if,lif,plif}_forward    -> (spike_seq, v_seq, v_last, h_seq)
    sj::hip_multistep_{if,lif,plif}_inference  -> (spike_seq, v_seq, v_last)
    sj::hip_multistep_{if,lif,plif}_backward   -> (grad_x_seq, grad_v_init[, grad_k])
    sj::hip_multistep_{if,lif,plif}_inference_packed -> (spike_bits, v_seq, v_last)
    sj::hip_multistep_qif_{forward,inference,backward}   the quadratic integrate-and-fire neuron, same outputs
    sj::hip_multistep_eif_{forward,inference,backward}   the exponential integrate-and-fire neuron
    sj::hip_multistep_ilif_{forward,inference,backward}  the integer-valued LIF: spike_seq holds counts 0..D

The ``_packed`` ops write the spikes bit-packed (uint8, ``T*N/8`` bytes, the layout of
``bit_spike_compress`` on the dense spike tensor) straight from the neuron kernel; they need ``N % 8 == 0``.

All tensors are viewed as ``[T, N]``; ``v_seq`` is an empty tensor when ``store_v_seq`` is false
(the kernel then writes only ``v_last``).  With ``recompute`` the forward writes no ``h_seq`` (an empty
tensor is returned) and autograd keeps ``x_seq`` and ``v_init`` instead; the backward then replays the
forward inside the kernel (``sjhip_neuron_backward_recompute``), which removes the forward's largest write.  ``Optional[float]`` is not expressible in an operator
schema, so soft reset is a bool next to a dummy ``v_reset`` as in the reference (lif.py:342-343).
The ops run on ROCm tensors only and raise otherwise; there is no fallback path.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import library as L

__all__ = [
    "hip_multistep_if_forward", "hip_multistep_if_inference", "hip_multistep_if_backward",
    "hip_multistep_lif_forward", "hip_multistep_lif_inference", "hip_multistep_lif_backward",
    "hip_multistep_plif_forward", "hip_multistep_plif_inference", "hip_multistep_plif_backward",
    "hip_multistep_if_inference_packed", "hip_multistep_lif_inference_packed", "hip_multistep_plif_inference_packed",
    "packed_supported",
    "hip_multistep_qif_forward", "hip_multistep_qif_inference", "hip_multistep_qif_backward",
    "hip_multistep_ilif_forward", "hip_multistep_ilif_inference", "hip_multistep_ilif_backward",
    "hip_multistep_eif_forward", "hip_multistep_eif_inference", "hip_multistep_eif_backward",
]


_NO_EXTRA = (0.0, 0.0, 0.0)


def _params(tau: float, v_th: float, v_reset: float, sg_alpha: float, sg_id: int, flags: int,
            qif: tuple[float, float, float] = _NO_EXTRA, levels: tuple[float, float, float] = _NO_EXTRA
            ) -> L.NeuronParams:
    """``qif`` is (v_rest, v_c, a0) of the quadratic neuron, ``levels`` is (level_max, grad_min, grad_max) of the
    integer-valued LIF; both unused by the others."""
    return L.NeuronParams(tau, v_th, v_reset, sg_alpha, sg_id, flags, *qif, *levels)


def _flags(soft_reset: bool, detach_reset: bool, decay_input: bool, mode_flags: int) -> int:
    f = int(mode_flags) & (L.FLAG_FP32_STATE | L.FLAG_RECIPROCAL_TAU | L.FLAG_ATOMIC_REDUCE)
    if soft_reset:
        f |= L.FLAG_SOFT_RESET
    if detach_reset:
        f |= L.FLAG_DETACH_RESET
    if decay_input:
        f |= L.FLAG_DECAY_INPUT
    return f


def _check_inputs(x_seq: torch.Tensor, v_init: torch.Tensor) -> None:
    L.require_device_tensor("x_seq", x_seq)
    L.require_device_tensor("v_init", v_init)
    if x_seq.dim() != 2:
        raise ValueError(f"x_seq must be [T, N], got shape {tuple(x_seq.shape)}")
    if v_init.shape != x_seq.shape[1:]:
        raise ValueError(f"v_init shape {tuple(v_init.shape)} does not match x_seq[0] {tuple(x_seq.shape[1:])}")
    if v_init.dtype != x_seq.dtype:
        raise ValueError(f"v_init dtype {v_init.dtype} != x_seq dtype {x_seq.dtype}")
    if x_seq.shape[0] < 1 or x_seq.shape[1] < 1:
        raise ValueError(f"x_seq must have T >= 1 and N >= 1, got shape {tuple(x_seq.shape)}")


def _is_broadcast_state(v: torch.Tensor) -> bool:
    """An expanded one-element tensor (every stride 0): what a node passes while its state is still the
    scalar reset value.  The kernels then read that one element instead of an [N] tensor."""
    return v.numel() > 1 and all(st == 0 for st in v.stride())


def _state_arg(v_init: torch.Tensor, align: bool) -> tuple[torch.Tensor, int]:
    """(tensor to keep alive, SJHIP_FLAG_V_INIT_BROADCAST or 0)."""
    if _is_broadcast_state(v_init):
        return v_init, L.FLAG_V_INIT_BROADCAST
    return (L.aligned16(v_init) if align else v_init.contiguous()), 0


def _k_pointer(k: Optional[torch.Tensor], ref: torch.Tensor) -> tuple[Optional[torch.Tensor], Optional[int]]:
    if k is None:
        return None, None
    L.require_device_tensor("k", k)
    k = k.detach().to(dtype=torch.float32, device=ref.device).reshape(1).contiguous()
    return k, k.data_ptr()


def _chunks(T: int, chunk: int) -> list[tuple[int, int]]:
    """Row ranges ``[t0, t1)`` of a sequence cut into pieces of at most ``chunk`` steps (one piece for ``chunk <= 0``)."""
    if chunk <= 0 or T <= chunk:
        return [(0, T)]
    return [(t0, min(t0 + chunk, T)) for t0 in range(0, T, chunk)]


def _run_forward(neuron: int, x_seq: torch.Tensor, v_init: torch.Tensor, k: Optional[torch.Tensor],
                 tau: float, v_th: float, v_reset: float, flags: int, store_v_seq: bool,
                 save_h: bool, qif: tuple[float, float, float] = _NO_EXTRA,
                 levels: tuple[float, float, float] = _NO_EXTRA, chunk: int = 0
                 ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """``(spike_seq, v_seq, v_last, h_seq)``.  With ``chunk > 0`` (and no ``h_seq``) a sequence longer than ``chunk``
    runs as pieces of ``chunk`` steps inside one launch, and the fourth result holds the state after every piece but
    the last, ``[pieces - 1, N]``: the checkpoints from which the backward replays piece by piece."""
    _check_inputs(x_seq, v_init)
    dtype = L.dtype_id(x_seq.dtype)
    T, N = x_seq.shape
    pieces = len(_chunks(T, 0 if save_h else chunk))
    x_seq = L.aligned16(x_seq) if pieces > 1 else x_seq.contiguous()
    v_init, broadcast = _state_arg(v_init, pieces > 1)
    spike_seq = torch.empty_like(x_seq)
    v_seq = torch.empty_like(x_seq) if store_v_seq else x_seq.new_empty((0,))
    v_last = x_seq.new_empty((N,))
    h_seq = torch.empty_like(x_seq) if save_h else None
    # a state kept in fp32 beside 16-bit storage is checkpointed in fp32
    ck_dtype = torch.float32 if flags & L.FLAG_FP32_STATE else x_seq.dtype
    checkpoints = x_seq.new_empty((pieces - 1, N), dtype=ck_dtype) if pieces > 1 else None
    k_keep, k_ptr = _k_pointer(k, x_seq)
    params = _params(tau, v_th, v_reset, 0.0, 0, flags | broadcast, qif, levels)
    lib = L.load()
    with torch.cuda.device(x_seq.device):
        stream = L.current_stream_ptr(x_seq.device)
        if pieces > 1:
            rc = lib.sjhip_neuron_forward_pieces(
                neuron, dtype, ctypes.byref(params), T, N, chunk,
                x_seq.data_ptr(), v_init.data_ptr(), k_ptr,
                spike_seq.data_ptr(), v_seq.data_ptr() if store_v_seq else None, v_last.data_ptr(),
                checkpoints.data_ptr(), stream,
            )
        else:
            rc = lib.sjhip_neuron_forward(
                neuron, dtype, ctypes.byref(params), T, N,
                x_seq.data_ptr(), v_init.data_ptr(), k_ptr,
                spike_seq.data_ptr(), v_seq.data_ptr() if store_v_seq else None, v_last.data_ptr(),
                h_seq.data_ptr() if save_h else None, stream,
            )
    L.check(rc, "neuron_forward")
    del k_keep
    return spike_seq, v_seq, v_last, (h_seq if checkpoints is None else checkpoints)


def packed_supported(n_neurons: int) -> bool:
    """The packed-spike forward needs every time step to start on a byte."""
    return n_neurons % 8 == 0


def _run_forward_packed(neuron: int, x_seq: torch.Tensor, v_init: torch.Tensor, k: Optional[torch.Tensor],
                        tau: float, v_th: float, v_reset: float, flags: int, store_v_seq: bool
                        ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _check_inputs(x_seq, v_init)
    dtype = L.dtype_id(x_seq.dtype)
    x_seq = x_seq.contiguous()
    v_init, broadcast = _state_arg(v_init, False)
    T, N = x_seq.shape
    if not packed_supported(N):
        raise NotImplementedError(f"packed spike output needs N % 8 == 0, got N={N}")
    spike_bits = torch.empty((T * N // 8,), dtype=torch.uint8, device=x_seq.device)
    v_seq = torch.empty_like(x_seq) if store_v_seq else x_seq.new_empty((0,))
    v_last = x_seq.new_empty((N,))
    k_keep, k_ptr = _k_pointer(k, x_seq)
    params = _params(tau, v_th, v_reset, 0.0, 0, flags | broadcast)
    with torch.cuda.device(x_seq.device):
        rc = L.load().sjhip_neuron_forward_packed(
            neuron, dtype, ctypes.byref(params), T, N,
            x_seq.data_ptr(), v_init.data_ptr(), k_ptr,
            spike_bits.data_ptr(), v_seq.data_ptr() if store_v_seq else None, v_last.data_ptr(),
            L.current_stream_ptr(x_seq.device),
        )
    L.check(rc, "neuron_forward_packed")
    del k_keep
    return spike_bits, v_seq, v_last


def _fake_forward_packed(x_seq, v_init, store_v_seq):
    return (x_seq.new_empty((x_seq.shape[0] * x_seq.shape[1] // 8,), dtype=torch.uint8),
            x_seq.new_empty(x_seq.shape) if store_v_seq else x_seq.new_empty((0,)),
            v_init.new_empty(v_init.shape))


def _forward_outputs(out, x_seq: torch.Tensor):
    """custom ops return tensors only: an unsaved h_seq becomes an empty tensor."""
    s, v_seq, v_last, h = out
    return s, v_seq, v_last, (h if h is not None else x_seq.new_empty((0,)))


def _run_backward(neuron: int, grad_spike_seq: Optional[torch.Tensor], grad_v_seq: Optional[torch.Tensor],
                  grad_v_last: Optional[torch.Tensor], h_seq: torch.Tensor, x_seq: Optional[torch.Tensor],
                  v_init: Optional[torch.Tensor], k: Optional[torch.Tensor], tau: float, v_th: float,
                  v_reset: float, flags: int, sg_id: int, sg_alpha: float, need_grad_v_init: bool = True,
                  qif: tuple[float, float, float] = _NO_EXTRA, levels: tuple[float, float, float] = _NO_EXTRA,
                  chunk: int = 0, checkpoints: Optional[torch.Tensor] = None
                  ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """``(grad_x_seq, grad_v_init, grad_k)``.  ``x_seq`` given: the replaying backward; with ``chunk > 0`` and the
    forward's ``checkpoints`` a long sequence is walked piece by piece from the last to the first, each piece replayed
    from its checkpoint, the gradient of a piece's initial state being the ``grad_v_last`` of the piece before it."""
    recompute = x_seq is not None
    if not recompute and h_seq is None:
        raise ValueError("backward needs h_seq, or x_seq and v_init to recompute it")
    if recompute:
        # replay path: every buffer must be 16-byte aligned for the 128-bit kernel
        h_seq = L.aligned16(x_seq)
        fix = L.aligned16
    else:
        h_seq = h_seq.contiguous()
        fix = lambda t: t.contiguous()
    broadcast = 0
    if v_init is not None:
        v_init, broadcast = _state_arg(v_init, recompute)
    L.require_device_tensor("h_seq", h_seq)
    dtype = L.dtype_id(h_seq.dtype)
    T, N = h_seq.shape
    pieces = len(_chunks(T, chunk if (recompute and checkpoints is not None) else 0))
    if grad_spike_seq is not None:  # None (a loss on v alone): the kernels read nothing in its place
        grad_spike_seq = fix(grad_spike_seq.to(h_seq.dtype))
    if grad_v_seq is not None:
        grad_v_seq = fix(grad_v_seq.to(h_seq.dtype))
    if grad_v_last is not None:
        grad_v_last = fix(grad_v_last.to(h_seq.dtype))
    grad_x_seq = torch.empty_like(h_seq)
    # a state that needs no gradient (the usual case: it was the reset value) costs no [N] write
    grad_v_init = h_seq.new_empty((N,) if need_grad_v_init else (0,))
    grad_k = workspace = None
    k_keep, k_ptr = _k_pointer(k, h_seq)
    if neuron == L.NEURON_PLIF:
        if flags & L.FLAG_ATOMIC_REDUCE:
            grad_k = torch.zeros((), dtype=torch.float32, device=h_seq.device)
        else:
            grad_k = torch.empty((), dtype=torch.float32, device=h_seq.device)
            workspace = torch.empty((L.load().sjhip_plif_workspace_floats(dtype, N),), dtype=torch.float32,
                                    device=h_seq.device)
    needs_state = neuron in (L.NEURON_PLIF, L.NEURON_QIF, L.NEURON_EIF)
    params = _params(tau, v_th, v_reset, sg_alpha, sg_id, flags | broadcast, qif, levels)
    carry_out = grad_v_init.data_ptr() if need_grad_v_init else None
    lib = L.load()
    with torch.cuda.device(h_seq.device):
        stream = L.current_stream_ptr(h_seq.device)
        if pieces > 1:
            rc = lib.sjhip_neuron_backward_recompute_pieces(
                neuron, dtype, ctypes.byref(params), T, N, chunk,
                h_seq.data_ptr(), v_init.data_ptr(), k_ptr, L.aligned16(checkpoints).data_ptr(),
                L.ptr(grad_spike_seq), L.ptr(grad_v_seq), L.ptr(grad_v_last),
                grad_x_seq.data_ptr(), carry_out, L.ptr(grad_k), L.ptr(workspace), stream,
            )
        elif recompute:
            rc = lib.sjhip_neuron_backward_recompute(
                neuron, dtype, ctypes.byref(params), T, N,
                h_seq.data_ptr(), v_init.data_ptr(), k_ptr,
                L.ptr(grad_spike_seq), L.ptr(grad_v_seq), L.ptr(grad_v_last),
                grad_x_seq.data_ptr(), carry_out, L.ptr(grad_k), L.ptr(workspace), stream,
            )
        else:
            rc = lib.sjhip_neuron_backward(
                neuron, dtype, ctypes.byref(params), T, N,
                L.ptr(grad_spike_seq), L.ptr(grad_v_seq), L.ptr(grad_v_last), h_seq.data_ptr(),
                L.ptr(v_init) if needs_state else None, k_ptr,
                grad_x_seq.data_ptr(), carry_out, L.ptr(grad_k), L.ptr(workspace), stream,
            )
    L.check(rc, "neuron_backward_recompute" if recompute else "neuron_backward")
    del k_keep
    return grad_x_seq, grad_v_init, grad_k


def _fake_forward(x_seq, v_init, store_v_seq, with_h, recompute=False):
    outs = [
        x_seq.new_empty(x_seq.shape),
        x_seq.new_empty(x_seq.shape) if store_v_seq else x_seq.new_empty((0,)),
        v_init.new_empty(v_init.shape),
    ]
    if with_h:
        outs.append(x_seq.new_empty((0,)) if recompute else x_seq.new_empty(x_seq.shape))
    return tuple(outs)


def _saved_for_backward(ctx, recompute: bool, x_seq, v_init, h_seq, *extra):
    """h path keeps h_seq; replay path keeps the op's own inputs x_seq and v_init."""
    ctx.recompute = recompute
    if recompute:
        ctx.save_for_backward(x_seq, v_init, *extra)
    else:
        ctx.save_for_backward(h_seq, *extra)


def _none_if_empty_grad(g: Optional[torch.Tensor], store_v_seq: bool) -> Optional[torch.Tensor]:
    return g if (store_v_seq and g is not None) else None


# =================================================================================================
# IF
# =================================================================================================
@torch.library.custom_op("sj::hip_multistep_if_forward", mutates_args=())
def hip_multistep_if_forward(x_seq: torch.Tensor, v_init: torch.Tensor, v_th: float, v_reset: float,
                             soft_reset: bool, detach_reset: bool, sg_id: int, sg_alpha: float,
                             store_v_seq: bool, mode_flags: int, recompute: bool
                             ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, detach_reset, False, mode_flags)
    return _forward_outputs(_run_forward(L.NEURON_IF, x_seq, v_init, None, 0.0, v_th, v_reset, flags, store_v_seq,
                                         not recompute), x_seq)


@hip_multistep_if_forward.register_fake
def _(x_seq, v_init, v_th, v_reset, soft_reset, detach_reset, sg_id, sg_alpha, store_v_seq, mode_flags, recompute):
    return _fake_forward(x_seq, v_init, store_v_seq, True, recompute)


@torch.library.custom_op("sj::hip_multistep_if_inference", mutates_args=())
def hip_multistep_if_inference(x_seq: torch.Tensor, v_init: torch.Tensor, v_th: float, v_reset: float,
                               soft_reset: bool, store_v_seq: bool, mode_flags: int
                               ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, False, False, mode_flags)
    return _run_forward(L.NEURON_IF, x_seq, v_init, None, 0.0, v_th, v_reset, flags, store_v_seq, False)[:3]


@hip_multistep_if_inference.register_fake
def _(x_seq, v_init, v_th, v_reset, soft_reset, store_v_seq, mode_flags):
    return _fake_forward(x_seq, v_init, store_v_seq, False)


@torch.library.custom_op("sj::hip_multistep_if_backward", mutates_args=())
def hip_multistep_if_backward(grad_spike_seq: Optional[torch.Tensor], grad_v_seq: Optional[torch.Tensor],
                              grad_v_last: Optional[torch.Tensor], h_seq: Optional[torch.Tensor],
                              x_seq: Optional[torch.Tensor], v_init: Optional[torch.Tensor], v_th: float,
                              v_reset: float, soft_reset: bool, detach_reset: bool, sg_id: int,
                              sg_alpha: float, mode_flags: int, need_grad_v_init: bool = True
                              ) -> tuple[torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, detach_reset, False, mode_flags)
    gx, gvi, _ = _run_backward(L.NEURON_IF, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, None,
                               0.0, v_th, v_reset, flags, sg_id, sg_alpha, need_grad_v_init)
    return gx, gvi


@hip_multistep_if_backward.register_fake
def _(grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, v_th, v_reset, soft_reset, detach_reset,
      sg_id, sg_alpha, mode_flags, need_grad_v_init=True):
    ref = h_seq if h_seq is not None else x_seq
    return torch.empty_like(ref), ref.new_empty(ref.shape[1:] if need_grad_v_init else (0,))


def _if_setup_context(ctx, inputs, output):
    (x_seq, v_init, v_th, v_reset, soft_reset, detach_reset, sg_id, sg_alpha, store_v_seq, mode_flags,
     recompute) = inputs
    _saved_for_backward(ctx, recompute, x_seq, v_init, output[3])
    ctx.scalars = (v_th, v_reset, soft_reset, detach_reset, sg_id, sg_alpha, mode_flags)
    ctx.store_v_seq = store_v_seq
    ctx.set_materialize_grads(False)


def _split_saved(ctx):
    """(h_seq, x_seq, v_init, extra...) from what _saved_for_backward stored."""
    saved = ctx.saved_tensors
    if ctx.recompute:
        return (None, saved[0], saved[1]) + tuple(saved[2:])
    return (saved[0], None, None) + tuple(saved[1:])


def _if_autograd_backward(ctx, grad_spike_seq, grad_v_seq, grad_v_last, grad_h_seq):
    del grad_h_seq
    h_seq, x_seq, v_init = _split_saved(ctx)
    v_th, v_reset, soft_reset, detach_reset, sg_id, sg_alpha, mode_flags = ctx.scalars
    need = bool(ctx.needs_input_grad[1])
    gx, gvi = hip_multistep_if_backward(
        grad_spike_seq, _none_if_empty_grad(grad_v_seq, ctx.store_v_seq), grad_v_last, h_seq, x_seq, v_init,
        v_th, v_reset, soft_reset, detach_reset, sg_id, sg_alpha, mode_flags, need)
    return gx, (gvi if need else None), None, None, None, None, None, None, None, None, None


torch.library.register_autograd("sj::hip_multistep_if_forward", _if_autograd_backward,
                                setup_context=_if_setup_context)


# =================================================================================================
# LIF
# =================================================================================================
@torch.library.custom_op("sj::hip_multistep_lif_forward", mutates_args=())
def hip_multistep_lif_forward(x_seq: torch.Tensor, v_init: torch.Tensor, v_th: float, v_reset: float,
                              soft_reset: bool, detach_reset: bool, tau: float, decay_input: bool,
                              sg_id: int, sg_alpha: float, store_v_seq: bool, mode_flags: int,
                              recompute: bool
                              ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, detach_reset, decay_input, mode_flags)
    return _forward_outputs(_run_forward(L.NEURON_LIF, x_seq, v_init, None, tau, v_th, v_reset, flags, store_v_seq,
                                         not recompute), x_seq)


@hip_multistep_lif_forward.register_fake
def _(x_seq, v_init, v_th, v_reset, soft_reset, detach_reset, tau, decay_input, sg_id, sg_alpha,
      store_v_seq, mode_flags, recompute):
    return _fake_forward(x_seq, v_init, store_v_seq, True, recompute)


@torch.library.custom_op("sj::hip_multistep_lif_inference", mutates_args=())
def hip_multistep_lif_inference(x_seq: torch.Tensor, v_init: torch.Tensor, v_th: float, v_reset: float,
                                soft_reset: bool, tau: float, decay_input: bool, store_v_seq: bool,
                                mode_flags: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, False, decay_input, mode_flags)
    return _run_forward(L.NEURON_LIF, x_seq, v_init, None, tau, v_th, v_reset, flags, store_v_seq, False)[:3]


@hip_multistep_lif_inference.register_fake
def _(x_seq, v_init, v_th, v_reset, soft_reset, tau, decay_input, store_v_seq, mode_flags):
    return _fake_forward(x_seq, v_init, store_v_seq, False)


@torch.library.custom_op("sj::hip_multistep_lif_backward", mutates_args=())
def hip_multistep_lif_backward(grad_spike_seq: Optional[torch.Tensor], grad_v_seq: Optional[torch.Tensor],
                               grad_v_last: Optional[torch.Tensor], h_seq: Optional[torch.Tensor],
                               x_seq: Optional[torch.Tensor], v_init: Optional[torch.Tensor], v_th: float,
                               v_reset: float, soft_reset: bool, detach_reset: bool, tau: float,
                               decay_input: bool, sg_id: int, sg_alpha: float, mode_flags: int,
                               need_grad_v_init: bool = True) -> tuple[torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, detach_reset, decay_input, mode_flags)
    gx, gvi, _ = _run_backward(L.NEURON_LIF, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, None,
                               tau, v_th, v_reset, flags, sg_id, sg_alpha, need_grad_v_init)
    return gx, gvi


@hip_multistep_lif_backward.register_fake
def _(grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, v_th, v_reset, soft_reset, detach_reset,
      tau, decay_input, sg_id, sg_alpha, mode_flags, need_grad_v_init=True):
    ref = h_seq if h_seq is not None else x_seq
    return torch.empty_like(ref), ref.new_empty(ref.shape[1:] if need_grad_v_init else (0,))


def _lif_setup_context(ctx, inputs, output):
    (x_seq, v_init, v_th, v_reset, soft_reset, detach_reset, tau, decay_input, sg_id, sg_alpha, store_v_seq,
     mode_flags, recompute) = inputs
    _saved_for_backward(ctx, recompute, x_seq, v_init, output[3])
    ctx.scalars = (v_th, v_reset, soft_reset, detach_reset, tau, decay_input, sg_id, sg_alpha, mode_flags)
    ctx.store_v_seq = store_v_seq
    ctx.set_materialize_grads(False)


def _lif_autograd_backward(ctx, grad_spike_seq, grad_v_seq, grad_v_last, grad_h_seq):
    del grad_h_seq
    h_seq, x_seq, v_init = _split_saved(ctx)
    need = bool(ctx.needs_input_grad[1])
    gx, gvi = hip_multistep_lif_backward(
        grad_spike_seq, _none_if_empty_grad(grad_v_seq, ctx.store_v_seq), grad_v_last, h_seq, x_seq, v_init,
        *ctx.scalars, need)
    return gx, (gvi if need else None), None, None, None, None, None, None, None, None, None, None, None


torch.library.register_autograd("sj::hip_multistep_lif_forward", _lif_autograd_backward,
                                setup_context=_lif_setup_context)


# =================================================================================================
# PLIF: k = sigmoid(w) is a 0-dim fp32 tensor on the device; the kernels read it from memory, so no
# host synchronisation happens (the reference's Triton path calls r_tau.item(), plif.py:666).
# =================================================================================================
@torch.library.custom_op("sj::hip_multistep_plif_forward", mutates_args=())
def hip_multistep_plif_forward(x_seq: torch.Tensor, v_init: torch.Tensor, k: torch.Tensor, v_th: float,
                               v_reset: float, soft_reset: bool, detach_reset: bool, decay_input: bool,
                               sg_id: int, sg_alpha: float, store_v_seq: bool, mode_flags: int,
                               recompute: bool
                               ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, detach_reset, decay_input, mode_flags)
    return _forward_outputs(_run_forward(L.NEURON_PLIF, x_seq, v_init, k, 0.0, v_th, v_reset, flags, store_v_seq,
                                         not recompute), x_seq)


@hip_multistep_plif_forward.register_fake
def _(x_seq, v_init, k, v_th, v_reset, soft_reset, detach_reset, decay_input, sg_id, sg_alpha,
      store_v_seq, mode_flags, recompute):
    return _fake_forward(x_seq, v_init, store_v_seq, True, recompute)


@torch.library.custom_op("sj::hip_multistep_plif_inference", mutates_args=())
def hip_multistep_plif_inference(x_seq: torch.Tensor, v_init: torch.Tensor, k: torch.Tensor, v_th: float,
                                 v_reset: float, soft_reset: bool, decay_input: bool, store_v_seq: bool,
                                 mode_flags: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, False, decay_input, mode_flags)
    return _run_forward(L.NEURON_PLIF, x_seq, v_init, k, 0.0, v_th, v_reset, flags, store_v_seq, False)[:3]


@hip_multistep_plif_inference.register_fake
def _(x_seq, v_init, k, v_th, v_reset, soft_reset, decay_input, store_v_seq, mode_flags):
    return _fake_forward(x_seq, v_init, store_v_seq, False)


@torch.library.custom_op("sj::hip_multistep_plif_backward", mutates_args=())
def hip_multistep_plif_backward(grad_spike_seq: Optional[torch.Tensor], grad_v_seq: Optional[torch.Tensor],
                                grad_v_last: Optional[torch.Tensor], h_seq: Optional[torch.Tensor],
                                x_seq: Optional[torch.Tensor], v_init: torch.Tensor, k: torch.Tensor,
                                v_th: float, v_reset: float,
                                soft_reset: bool, detach_reset: bool, decay_input: bool, sg_id: int,
                                sg_alpha: float, mode_flags: int, need_grad_v_init: bool = True
                                ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, detach_reset, decay_input, mode_flags)
    gx, gvi, gk = _run_backward(L.NEURON_PLIF, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, k,
                                0.0, v_th, v_reset, flags, sg_id, sg_alpha, need_grad_v_init)
    return gx, gvi, gk


@hip_multistep_plif_backward.register_fake
def _(grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, k, v_th, v_reset, soft_reset,
      detach_reset, decay_input, sg_id, sg_alpha, mode_flags, need_grad_v_init=True):
    ref = h_seq if h_seq is not None else x_seq
    return (torch.empty_like(ref), ref.new_empty(ref.shape[1:] if need_grad_v_init else (0,)),
            ref.new_empty((), dtype=torch.float32))


def _plif_setup_context(ctx, inputs, output):
    (x_seq, v_init, k, v_th, v_reset, soft_reset, detach_reset, decay_input, sg_id, sg_alpha, store_v_seq,
     mode_flags, recompute) = inputs
    ctx.recompute = recompute
    if recompute:
        ctx.save_for_backward(x_seq, v_init, k)
    else:
        ctx.save_for_backward(output[3], v_init, k)
    ctx.scalars = (v_th, v_reset, soft_reset, detach_reset, decay_input, sg_id, sg_alpha, mode_flags)
    ctx.store_v_seq = store_v_seq
    ctx.k_shape = k.shape
    ctx.k_dtype = k.dtype
    ctx.set_materialize_grads(False)


def _plif_autograd_backward(ctx, grad_spike_seq, grad_v_seq, grad_v_last, grad_h_seq):
    del grad_h_seq
    first, v_init, k = ctx.saved_tensors
    h_seq, x_seq = (None, first) if ctx.recompute else (first, None)
    need = bool(ctx.needs_input_grad[1])
    gx, gvi, gk = hip_multistep_plif_backward(
        grad_spike_seq, _none_if_empty_grad(grad_v_seq, ctx.store_v_seq), grad_v_last, h_seq, x_seq, v_init, k,
        *ctx.scalars, need)
    gk = gk.reshape(ctx.k_shape).to(ctx.k_dtype)
    return gx, (gvi if need else None), gk, None, None, None, None, None, None, None, None, None, None


torch.library.register_autograd("sj::hip_multistep_plif_forward", _plif_autograd_backward,
                                setup_context=_plif_setup_context)


# =================================================================================================
# Inference with bit-packed spike output (all three neurons)
# =================================================================================================
@torch.library.custom_op("sj::hip_multistep_if_inference_packed", mutates_args=())
def hip_multistep_if_inference_packed(x_seq: torch.Tensor, v_init: torch.Tensor, v_th: float, v_reset: float,
                                      soft_reset: bool, store_v_seq: bool, mode_flags: int
                                      ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, False, False, mode_flags)
    return _run_forward_packed(L.NEURON_IF, x_seq, v_init, None, 0.0, v_th, v_reset, flags, store_v_seq)


@hip_multistep_if_inference_packed.register_fake
def _(x_seq, v_init, v_th, v_reset, soft_reset, store_v_seq, mode_flags):
    return _fake_forward_packed(x_seq, v_init, store_v_seq)


@torch.library.custom_op("sj::hip_multistep_lif_inference_packed", mutates_args=())
def hip_multistep_lif_inference_packed(x_seq: torch.Tensor, v_init: torch.Tensor, v_th: float, v_reset: float,
                                       soft_reset: bool, tau: float, decay_input: bool, store_v_seq: bool,
                                       mode_flags: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, False, decay_input, mode_flags)
    return _run_forward_packed(L.NEURON_LIF, x_seq, v_init, None, tau, v_th, v_reset, flags, store_v_seq)


@hip_multistep_lif_inference_packed.register_fake
def _(x_seq, v_init, v_th, v_reset, soft_reset, tau, decay_input, store_v_seq, mode_flags):
    return _fake_forward_packed(x_seq, v_init, store_v_seq)


@torch.library.custom_op("sj::hip_multistep_plif_inference_packed", mutates_args=())
def hip_multistep_plif_inference_packed(x_seq: torch.Tensor, v_init: torch.Tensor, k: torch.Tensor, v_th: float,
                                        v_reset: float, soft_reset: bool, decay_input: bool, store_v_seq: bool,
                                        mode_flags: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, False, decay_input, mode_flags)
    return _run_forward_packed(L.NEURON_PLIF, x_seq, v_init, k, 0.0, v_th, v_reset, flags, store_v_seq)


@hip_multistep_plif_inference_packed.register_fake
def _(x_seq, v_init, k, v_th, v_reset, soft_reset, decay_input, store_v_seq, mode_flags):
    return _fake_forward_packed(x_seq, v_init, store_v_seq)


# =================================================================================================
# QIF: h = v + (x + a0 (v - v_rest)(v - v_c)) / tau  (reference cuda_kernel/neuron_kernel/multi_step/qif.py)
# =================================================================================================
@torch.library.custom_op("sj::hip_multistep_qif_forward", mutates_args=())
def hip_multistep_qif_forward(x_seq: torch.Tensor, v_init: torch.Tensor, v_th: float, v_reset: float,
                              soft_reset: bool, detach_reset: bool, tau: float, v_rest: float, v_c: float,
                              a0: float, sg_id: int, sg_alpha: float, store_v_seq: bool, mode_flags: int,
                              recompute: bool
                              ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, detach_reset, True, mode_flags)
    return _forward_outputs(_run_forward(L.NEURON_QIF, x_seq, v_init, None, tau, v_th, v_reset, flags, store_v_seq,
                                         not recompute, (v_rest, v_c, a0)), x_seq)


@hip_multistep_qif_forward.register_fake
def _(x_seq, v_init, v_th, v_reset, soft_reset, detach_reset, tau, v_rest, v_c, a0, sg_id, sg_alpha, store_v_seq,
      mode_flags, recompute):
    return _fake_forward(x_seq, v_init, store_v_seq, True, recompute)


@torch.library.custom_op("sj::hip_multistep_qif_inference", mutates_args=())
def hip_multistep_qif_inference(x_seq: torch.Tensor, v_init: torch.Tensor, v_th: float, v_reset: float,
                                soft_reset: bool, tau: float, v_rest: float, v_c: float, a0: float,
                                store_v_seq: bool, mode_flags: int
                                ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, False, True, mode_flags)
    return _run_forward(L.NEURON_QIF, x_seq, v_init, None, tau, v_th, v_reset, flags, store_v_seq, False,
                        (v_rest, v_c, a0))[:3]


@hip_multistep_qif_inference.register_fake
def _(x_seq, v_init, v_th, v_reset, soft_reset, tau, v_rest, v_c, a0, store_v_seq, mode_flags):
    return _fake_forward(x_seq, v_init, store_v_seq, False)


@torch.library.custom_op("sj::hip_multistep_qif_backward", mutates_args=())
def hip_multistep_qif_backward(grad_spike_seq: Optional[torch.Tensor], grad_v_seq: Optional[torch.Tensor],
                               grad_v_last: Optional[torch.Tensor], h_seq: Optional[torch.Tensor],
                               x_seq: Optional[torch.Tensor], v_init: torch.Tensor, v_th: float,
                               v_reset: float, soft_reset: bool, detach_reset: bool, tau: float, v_rest: float,
                               v_c: float, a0: float, sg_id: int, sg_alpha: float, mode_flags: int,
                               need_grad_v_init: bool = True) -> tuple[torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, detach_reset, True, mode_flags)
    gx, gvi, _ = _run_backward(L.NEURON_QIF, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, None,
                               tau, v_th, v_reset, flags, sg_id, sg_alpha, need_grad_v_init, (v_rest, v_c, a0))
    return gx, gvi


@hip_multistep_qif_backward.register_fake
def _(grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, v_th, v_reset, soft_reset, detach_reset,
      tau, v_rest, v_c, a0, sg_id, sg_alpha, mode_flags, need_grad_v_init=True):
    ref = h_seq if h_seq is not None else x_seq
    return torch.empty_like(ref), ref.new_empty(ref.shape[1:] if need_grad_v_init else (0,))


def _qif_setup_context(ctx, inputs, output):
    (x_seq, v_init, v_th, v_reset, soft_reset, detach_reset, tau, v_rest, v_c, a0, sg_id, sg_alpha, store_v_seq,
     mode_flags, recompute) = inputs
    ctx.recompute = recompute
    # the state-dependent dh/dv needs v_init on both paths
    if recompute:
        ctx.save_for_backward(x_seq, v_init)
    else:
        ctx.save_for_backward(output[3], v_init)
    ctx.scalars = (v_th, v_reset, soft_reset, detach_reset, tau, v_rest, v_c, a0, sg_id, sg_alpha, mode_flags)
    ctx.store_v_seq = store_v_seq
    ctx.set_materialize_grads(False)


def _qif_autograd_backward(ctx, grad_spike_seq, grad_v_seq, grad_v_last, grad_h_seq):
    del grad_h_seq
    first, v_init = ctx.saved_tensors
    h_seq, x_seq = (None, first) if ctx.recompute else (first, None)
    need = bool(ctx.needs_input_grad[1])
    gx, gvi = hip_multistep_qif_backward(
        grad_spike_seq, _none_if_empty_grad(grad_v_seq, ctx.store_v_seq), grad_v_last, h_seq, x_seq, v_init,
        *ctx.scalars, need)
    return (gx, (gvi if need else None)) + (None,) * 13


torch.library.register_autograd("sj::hip_multistep_qif_forward", _qif_autograd_backward,
                                setup_context=_qif_setup_context)


# =================================================================================================
# EIF: h = v + (x + v_rest - v + delta_T exp((v - theta_rh) / delta_T)) / tau
# (reference cuda_kernel/neuron_kernel/multi_step/eif.py); theta_rh and delta_T travel in the parameter fields v_c and a0
# =================================================================================================
@torch.library.custom_op("sj::hip_multistep_eif_forward", mutates_args=())
def hip_multistep_eif_forward(x_seq: torch.Tensor, v_init: torch.Tensor, v_th: float, v_reset: float,
                              soft_reset: bool, detach_reset: bool, tau: float, v_rest: float, theta_rh: float,
                              delta_t: float, sg_id: int, sg_alpha: float, store_v_seq: bool, mode_flags: int,
                              recompute: bool
                              ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, detach_reset, True, mode_flags)
    return _forward_outputs(_run_forward(L.NEURON_EIF, x_seq, v_init, None, tau, v_th, v_reset, flags, store_v_seq,
                                         not recompute, (v_rest, theta_rh, delta_t)), x_seq)


@hip_multistep_eif_forward.register_fake
def _(x_seq, v_init, v_th, v_reset, soft_reset, detach_reset, tau, v_rest, theta_rh, delta_t, sg_id, sg_alpha, store_v_seq,
      mode_flags, recompute):
    return _fake_forward(x_seq, v_init, store_v_seq, True, recompute)


@torch.library.custom_op("sj::hip_multistep_eif_inference", mutates_args=())
def hip_multistep_eif_inference(x_seq: torch.Tensor, v_init: torch.Tensor, v_th: float, v_reset: float,
                                soft_reset: bool, tau: float, v_rest: float, theta_rh: float, delta_t: float,
                                store_v_seq: bool, mode_flags: int
                                ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, False, True, mode_flags)
    return _run_forward(L.NEURON_EIF, x_seq, v_init, None, tau, v_th, v_reset, flags, store_v_seq, False,
                        (v_rest, theta_rh, delta_t))[:3]


@hip_multistep_eif_inference.register_fake
def _(x_seq, v_init, v_th, v_reset, soft_reset, tau, v_rest, theta_rh, delta_t, store_v_seq, mode_flags):
    return _fake_forward(x_seq, v_init, store_v_seq, False)


@torch.library.custom_op("sj::hip_multistep_eif_backward", mutates_args=())
def hip_multistep_eif_backward(grad_spike_seq: Optional[torch.Tensor], grad_v_seq: Optional[torch.Tensor],
                               grad_v_last: Optional[torch.Tensor], h_seq: Optional[torch.Tensor],
                               x_seq: Optional[torch.Tensor], v_init: torch.Tensor, v_th: float,
                               v_reset: float, soft_reset: bool, detach_reset: bool, tau: float, v_rest: float,
                               theta_rh: float, delta_t: float, sg_id: int, sg_alpha: float, mode_flags: int,
                               need_grad_v_init: bool = True) -> tuple[torch.Tensor, torch.Tensor]:
    flags = _flags(soft_reset, detach_reset, True, mode_flags)
    gx, gvi, _ = _run_backward(L.NEURON_EIF, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, None,
                               tau, v_th, v_reset, flags, sg_id, sg_alpha, need_grad_v_init, (v_rest, theta_rh, delta_t))
    return gx, gvi


@hip_multistep_eif_backward.register_fake
def _(grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, v_th, v_reset, soft_reset, detach_reset,
      tau, v_rest, theta_rh, delta_t, sg_id, sg_alpha, mode_flags, need_grad_v_init=True):
    ref = h_seq if h_seq is not None else x_seq
    return torch.empty_like(ref), ref.new_empty(ref.shape[1:] if need_grad_v_init else (0,))


def _eif_setup_context(ctx, inputs, output):
    (x_seq, v_init, v_th, v_reset, soft_reset, detach_reset, tau, v_rest, theta_rh, delta_t, sg_id, sg_alpha, store_v_seq,
     mode_flags, recompute) = inputs
    ctx.recompute = recompute
    # the state-dependent dh/dv needs v_init on both paths
    if recompute:
        ctx.save_for_backward(x_seq, v_init)
    else:
        ctx.save_for_backward(output[3], v_init)
    ctx.scalars = (v_th, v_reset, soft_reset, detach_reset, tau, v_rest, theta_rh, delta_t, sg_id, sg_alpha, mode_flags)
    ctx.store_v_seq = store_v_seq
    ctx.set_materialize_grads(False)


def _eif_autograd_backward(ctx, grad_spike_seq, grad_v_seq, grad_v_last, grad_h_seq):
    del grad_h_seq
    first, v_init = ctx.saved_tensors
    h_seq, x_seq = (None, first) if ctx.recompute else (first, None)
    need = bool(ctx.needs_input_grad[1])
    gx, gvi = hip_multistep_eif_backward(
        grad_spike_seq, _none_if_empty_grad(grad_v_seq, ctx.store_v_seq), grad_v_last, h_seq, x_seq, v_init,
        *ctx.scalars, need)
    return (gx, (gvi if need else None)) + (None,) * 13


torch.library.register_autograd("sj::hip_multistep_eif_forward", _eif_autograd_backward,
                                setup_context=_eif_setup_context)


# =================================================================================================
# ILIF: h = v - v / tau + x,  c = rint(clamp(h / v_th, 0, D)),  v' = h - c v_th
# (reference triton_kernel/neuron_kernel/ilif.py:556-726; the op there takes decay = 1 - 1/tau, these take tau
# because the kernels charge in the torch backend's own arithmetic form)
# =================================================================================================
@torch.library.custom_op("sj::hip_multistep_ilif_forward", mutates_args=())
def hip_multistep_ilif_forward(x_seq: torch.Tensor, v_init: torch.Tensor, tau: float, v_th: float,
                               max_spike_count: int, grad_min: float, grad_max: float, detach_reset: bool,
                               store_v_seq: bool, mode_flags: int, recompute: bool
                               ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(True, detach_reset, False, mode_flags)
    return _forward_outputs(_run_forward(L.NEURON_ILIF, x_seq, v_init, None, tau, v_th, 0.0, flags, store_v_seq,
                                         not recompute, levels=(float(max_spike_count), grad_min, grad_max)), x_seq)


@hip_multistep_ilif_forward.register_fake
def _(x_seq, v_init, tau, v_th, max_spike_count, grad_min, grad_max, detach_reset, store_v_seq, mode_flags,
      recompute):
    return _fake_forward(x_seq, v_init, store_v_seq, True, recompute)


@torch.library.custom_op("sj::hip_multistep_ilif_inference", mutates_args=())
def hip_multistep_ilif_inference(x_seq: torch.Tensor, v_init: torch.Tensor, tau: float, v_th: float,
                                 max_spike_count: int, store_v_seq: bool, mode_flags: int
                                 ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    flags = _flags(True, False, False, mode_flags)
    return _run_forward(L.NEURON_ILIF, x_seq, v_init, None, tau, v_th, 0.0, flags, store_v_seq, False,
                        levels=(float(max_spike_count), 0.0, 0.0))[:3]


@hip_multistep_ilif_inference.register_fake
def _(x_seq, v_init, tau, v_th, max_spike_count, store_v_seq, mode_flags):
    return _fake_forward(x_seq, v_init, store_v_seq, False)


@torch.library.custom_op("sj::hip_multistep_ilif_backward", mutates_args=())
def hip_multistep_ilif_backward(grad_spike_seq: Optional[torch.Tensor], grad_v_seq: Optional[torch.Tensor],
                                grad_v_last: Optional[torch.Tensor], h_seq: Optional[torch.Tensor],
                                x_seq: Optional[torch.Tensor], v_init: Optional[torch.Tensor], tau: float,
                                v_th: float, max_spike_count: int, grad_min: float, grad_max: float,
                                detach_reset: bool, mode_flags: int, need_grad_v_init: bool = True
                                ) -> tuple[torch.Tensor, torch.Tensor]:
    flags = _flags(True, detach_reset, False, mode_flags)
    gx, gvi, _ = _run_backward(L.NEURON_ILIF, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, None,
                               tau, v_th, 0.0, flags, L.SG_MULTI_LEVEL, 0.0, need_grad_v_init,
                               levels=(float(max_spike_count), grad_min, grad_max))
    return gx, gvi


@hip_multistep_ilif_backward.register_fake
def _(grad_spike_seq, grad_v_seq, grad_v_last, h_seq, x_seq, v_init, tau, v_th, max_spike_count, grad_min,
      grad_max, detach_reset, mode_flags, need_grad_v_init=True):
    ref = h_seq if h_seq is not None else x_seq
    return torch.empty_like(ref), ref.new_empty(ref.shape[1:] if need_grad_v_init else (0,))


def _ilif_setup_context(ctx, inputs, output):
    (x_seq, v_init, tau, v_th, max_spike_count, grad_min, grad_max, detach_reset, store_v_seq, mode_flags,
     recompute) = inputs
    _saved_for_backward(ctx, recompute, x_seq, v_init, output[3])
    ctx.scalars = (tau, v_th, max_spike_count, grad_min, grad_max, detach_reset, mode_flags)
    ctx.store_v_seq = store_v_seq
    ctx.set_materialize_grads(False)


def _ilif_autograd_backward(ctx, grad_spike_seq, grad_v_seq, grad_v_last, grad_h_seq):
    del grad_h_seq
    h_seq, x_seq, v_init = _split_saved(ctx)
    need = bool(ctx.needs_input_grad[1])
    gx, gvi = hip_multistep_ilif_backward(
        grad_spike_seq, _none_if_empty_grad(grad_v_seq, ctx.store_v_seq), grad_v_last, h_seq, x_seq, v_init,
        *ctx.scalars, need)
    return (gx, (gvi if need else None)) + (None,) * 9


torch.library.register_autograd("sj::hip_multistep_ilif_forward", _ilif_autograd_backward,
                                setup_context=_ilif_setup_context)


# =================================================================================================
# Eager entry: the same kernels without the operator dispatch
# =================================================================================================
class _EagerNeuron(torch.autograd.Function):
    """What the ``sj::hip_multistep_*_forward`` operators and their registered autograd do, as one plain
    ``autograd.Function`` for code that is not being traced: a call through the operator registry costs about
    55 us (forward) + 50 us (backward) of host time on top of the 12 us each launch takes, this about 15 + 30."""

    @staticmethod
    def forward(x_seq, v_init, k, spec):
        neuron, tau, v_th, v_reset, flags, _, _, store_v_seq, recompute, qif, levels, chunk = spec
        s, v_seq, v_last, kept = _run_forward(neuron, x_seq, v_init, k, tau, v_th, v_reset, flags, store_v_seq,
                                              not recompute, qif, levels, chunk)
        # kept: h_seq (saved-h route), the checkpoints of a sequence replayed piece by piece, or nothing
        return s, v_seq, v_last, (kept if kept is not None else x_seq.new_empty((0,)))

    @staticmethod
    def setup_context(ctx, inputs, output):
        x_seq, v_init, k, spec = inputs
        neuron, recompute = spec[0], spec[8]
        ctx.spec = spec
        # PLIF and QIF need the state before the first step in either backward; the replay needs it to start from
        keep_v_init = recompute or neuron in (L.NEURON_PLIF, L.NEURON_QIF, L.NEURON_EIF)
        ctx.save_for_backward(x_seq if recompute else output[3], v_init if keep_v_init else None, k,
                              output[3] if (recompute and output[3].numel() > 0) else None)
        ctx.mark_non_differentiable(output[3])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_spike_seq, grad_v_seq, grad_v_last, grad_h_seq):
        del grad_h_seq
        neuron, tau, v_th, v_reset, flags, sg_id, sg_alpha, store_v_seq, recompute, qif, levels, chunk = ctx.spec
        first, v_init, k, checkpoints = ctx.saved_tensors
        h_seq, x_seq = (None, first) if recompute else (first, None)
        need = bool(ctx.needs_input_grad[1])
        gx, gvi, gk = _run_backward(neuron, grad_spike_seq, _none_if_empty_grad(grad_v_seq, store_v_seq), grad_v_last,
                                    h_seq, x_seq, v_init, k, tau, v_th, v_reset, flags, sg_id, sg_alpha, need, qif, levels,
                                    chunk, checkpoints)
        if gk is not None:
            gk = gk.reshape(k.shape).to(k.dtype)
        return gx, (gvi if need else None), gk, None


def replay_chunk(dtype: torch.dtype, T: int, N: int, flags: int) -> int:
    """Steps per piece when a sequence of ``T`` steps should be replayed piece by piece in the backward, else 0: the
    replay is switched on, one piece of the configured length is a shape the replay kernel prefers, and the sequence
    is longer than that."""
    from ... import configure

    chunk = int(configure.hip_replay_chunk)
    if not configure.hip_backward_recompute or chunk <= 0 or T <= chunk:
        return 0
    return chunk if L.recompute_preferred(dtype, chunk, N, flags) else 0


def eager_multistep(neuron: int, x_seq: torch.Tensor, v_init: torch.Tensor, k: Optional[torch.Tensor], tau: float,
                    v_th: float, v_reset: float, flags: int, sg_id: int, sg_alpha: float, store_v_seq: bool,
                    recompute: bool, need_grad: bool, qif: tuple[float, float, float] = _NO_EXTRA,
                    levels: tuple[float, float, float] = _NO_EXTRA
                    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(spike_seq, v_seq, v_last)`` of any neuron kind for ``[T, N]`` / ``[N]`` inputs, outside a tracing
    compiler.  ``flags`` is the complete flag word (``_flags``); ``need_grad`` selects the training path (saves
    ``h_seq``, or ``x_seq`` and ``v_init`` with ``recompute``) or the inference path (saves nothing)."""
    if need_grad:
        chunk = 0
        if not recompute:
            # a sequence too long to replay in one piece (its h would not fit in LDS with enough resident wavefronts) is
            # replayed in pieces from checkpoints of the state, instead of saving and re-reading h_seq
            chunk = replay_chunk(x_seq.dtype, x_seq.shape[0], x_seq.shape[1], flags)
            recompute = chunk > 0
        spec = (neuron, tau, v_th, v_reset, flags, sg_id, sg_alpha, store_v_seq, recompute, qif, levels, chunk)
        return _EagerNeuron.apply(x_seq, v_init, k, spec)[:3]
    return _run_forward(neuron, x_seq.detach(), v_init.detach(), None if k is None else k.detach(), tau, v_th, v_reset,
                        flags, store_v_seq, False, qif, levels)[:3]
