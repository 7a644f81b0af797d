"""``torch.library`` operators for the spiking self-attention contraction on the matrix cores.

    sj::hip_ssa_forward(qkv [S, 3, H, Cph, L], scale)            -> out [S, H, Cph, L]
    sj::hip_ssa_backward(qkv, grad_out, scale)                    -> grad_qkv

``out = scale * (v @ k^T) @ q`` per (sample, head), the contraction of the reference's
``SpikingSelfAttention._ssa_kernel_torch`` (layer/attention.py:346-353).  qkv must hold binary spikes.
"""

from __future__ import annotations

import ctypes

import torch

from . import library as L

__all__ = ["hip_ssa_forward", "hip_ssa_backward", "ssa_supported"]


@torch.compiler.assume_constant_result
def ssa_supported(dtype: torch.dtype, channels_per_head: int, tokens: int) -> bool:
    """(asks the library; a constant of any traced graph, like the shapes it is asked about)"""
    try:
        did = L.dtype_id(dtype)
    except NotImplementedError:
        return False
    return bool(L.load().sjhip_ssa_supported(did, channels_per_head, tokens))


def _check(qkv: torch.Tensor) -> tuple[int, int, int, int]:
    L.require_device_tensor("qkv", qkv)
    if qkv.dim() != 5 or qkv.shape[1] != 3:
        raise ValueError(f"qkv must be [samples, 3, heads, channels_per_head, tokens], got {tuple(qkv.shape)}")
    samples, _, heads, cph, tokens = qkv.shape
    if not ssa_supported(qkv.dtype, cph, tokens):
        raise NotImplementedError(
            f"hip spiking self-attention supports fp32/fp16/bf16 with at most 64 channels per head and at most "
            f"256 tokens (one head's tiles must fit in LDS); got dtype={qkv.dtype}, channels_per_head={cph}, "
            f"tokens={tokens}. Use backend='torch'."
        )
    return samples, heads, cph, tokens


@torch.library.custom_op("sj::hip_ssa_forward", mutates_args=())
def hip_ssa_forward(qkv: torch.Tensor, scale: float) -> torch.Tensor:
    samples, heads, cph, tokens = _check(qkv)
    qkv = qkv.contiguous()
    out = qkv.new_empty((samples, heads, cph, tokens))
    with torch.cuda.device(qkv.device):
        rc = L.load().sjhip_ssa_forward(L.dtype_id(qkv.dtype), samples, heads, cph, tokens, scale, qkv.data_ptr(),
                                        out.data_ptr(), L.current_stream_ptr(qkv.device))
    L.check(rc, "ssa_forward")
    return out


@hip_ssa_forward.register_fake
def _(qkv, scale):
    return qkv.new_empty((qkv.shape[0], qkv.shape[2], qkv.shape[3], qkv.shape[4]))


@torch.library.custom_op("sj::hip_ssa_backward", mutates_args=())
def hip_ssa_backward(qkv: torch.Tensor, grad_out: torch.Tensor, scale: float) -> torch.Tensor:
    samples, heads, cph, tokens = _check(qkv)
    qkv = qkv.contiguous()
    grad_out = grad_out.to(qkv.dtype).contiguous()
    grad_qkv = torch.empty_like(qkv)
    with torch.cuda.device(qkv.device):
        rc = L.load().sjhip_ssa_backward(L.dtype_id(qkv.dtype), samples, heads, cph, tokens, scale, qkv.data_ptr(),
                                         grad_out.data_ptr(), grad_qkv.data_ptr(), L.current_stream_ptr(qkv.device))
    L.check(rc, "ssa_backward")
    return grad_qkv


@hip_ssa_backward.register_fake
def _(qkv, grad_out, scale):
    return torch.empty_like(qkv)


def _setup_context(ctx, inputs, output):
    qkv, scale = inputs
    ctx.save_for_backward(qkv)
    ctx.scale = scale


def _backward(ctx, grad_out):
    (qkv,) = ctx.saved_tensors
    return hip_ssa_backward(qkv, grad_out, ctx.scale), None


torch.library.register_autograd("sj::hip_ssa_forward", _backward, setup_context=_setup_context)


# =================================================================================================
# LIF -> contraction with the spikes kept bit-packed in between
# =================================================================================================
def ssa_packed_supported(dtype: torch.dtype, channels_per_head: int, tokens: int) -> bool:
    """The packed-operand contraction needs every head's tile to start on a byte."""
    return ssa_supported(dtype, channels_per_head, tokens) and (channels_per_head * tokens) % 8 == 0


def _ssa_packed(bits: torch.Tensor, grad_out, dtype: torch.dtype, samples: int, heads: int, cph: int, tokens: int,
                scale: float) -> torch.Tensor:
    """Forward (``grad_out is None``: returns out) or backward (returns grad_qkv) of the contraction on bit-packed q/k/v."""
    lib = L.load()
    with torch.cuda.device(bits.device):
        if grad_out is None:
            result = torch.empty((samples, heads, cph, tokens), dtype=dtype, device=bits.device)
            rc = lib.sjhip_ssa_forward_packed(L.dtype_id(dtype), samples, heads, cph, tokens, scale, bits.data_ptr(),
                                              result.data_ptr(), L.current_stream_ptr(bits.device))
        else:
            grad_out = grad_out.to(dtype).contiguous()
            result = torch.empty((samples, 3, heads, cph, tokens), dtype=dtype, device=bits.device)
            rc = lib.sjhip_ssa_backward_packed(L.dtype_id(dtype), samples, heads, cph, tokens, scale, bits.data_ptr(),
                                               grad_out.data_ptr(), result.data_ptr(), L.current_stream_ptr(bits.device))
    L.check(rc, "ssa_forward_packed" if grad_out is None else "ssa_backward_packed")
    return result


def ssa_lif_supported(channels_per_head: int, tokens: int) -> bool:
    """The contraction fused with the LIF behind it: fp32, bit-packed q / k / v, tokens a multiple of 4."""
    return ssa_packed_supported(torch.float32, channels_per_head, tokens) and tokens % 4 == 0


def _ssa_lif_forward(bits: torch.Tensor, v_init: torch.Tensor, params, T: int, B: int, heads: int, cph: int, tokens: int,
                     scale: float, save_h: bool):
    """``(spikes [T, B, heads, cph, tokens], h_seq or None, v_last [B, heads, cph, tokens])`` of the LIF that takes
    ``scale (V K^T) Q`` of the bit-packed spikes as its input; the contraction's output is never written."""
    spikes = torch.empty((T, B, heads, cph, tokens), dtype=torch.float32, device=bits.device)
    h_seq = torch.empty_like(spikes) if save_h else None
    v_last = torch.empty((B, heads, cph, tokens), dtype=torch.float32, device=bits.device)
    with torch.cuda.device(bits.device):
        rc = L.load().sjhip_ssa_lif_forward_packed(L.NEURON_LIF, ctypes.byref(params), T, B, heads, cph, tokens, scale,
                                                   bits.data_ptr(), v_init.data_ptr(), spikes.data_ptr(), L.ptr(h_seq),
                                                   v_last.data_ptr(), L.current_stream_ptr(bits.device))
    L.check(rc, "ssa_lif_forward_packed")
    return spikes, h_seq, v_last


def _ssa_lif_backward(bits: torch.Tensor, h_seq: torch.Tensor, grad_spikes, grad_v_last, params, T: int, B: int, heads: int,
                      cph: int, tokens: int, scale: float, need_grad_v_init: bool):
    """``(grad_qkv [T * B, 3, heads, cph, tokens], grad_v_init or None)``."""
    grad_qkv = torch.empty((T * B, 3, heads, cph, tokens), dtype=torch.float32, device=bits.device)
    grad_v_init = torch.empty((B, heads, cph, tokens), dtype=torch.float32, device=bits.device) if need_grad_v_init else None
    gs = L.aligned16(grad_spikes.to(torch.float32)) if grad_spikes is not None else None
    gvl = L.aligned16(grad_v_last.to(torch.float32)) if grad_v_last is not None else None
    with torch.cuda.device(bits.device):
        rc = L.load().sjhip_ssa_lif_backward_packed(L.NEURON_LIF, ctypes.byref(params), T, B, heads, cph, tokens, scale,
                                                    bits.data_ptr(), h_seq.data_ptr(), L.ptr(gs), L.ptr(gvl),
                                                    grad_qkv.data_ptr(), L.ptr(grad_v_init),
                                                    L.current_stream_ptr(bits.device))
    L.check(rc, "ssa_lif_backward_packed")
    return grad_qkv, grad_v_init


class _LifSsa(torch.autograd.Function):
    """``out = scale (V K^T) Q`` of the spikes a multi-step LIF fires from ``x_seq``, with those spikes existing only
    bit-packed: the LIF forward writes bits (``sjhip_neuron_forward_packed``), the contraction reads bits, and in the
    backward the contraction writes the dense spike gradient that the replaying LIF backward consumes.  Saves
    ``x_seq``, ``v_init`` and the bits (1/32 of the fp32 spike tensor)."""

    @staticmethod
    def forward(x_seq, v_init, spec):
        from . import neuron_kernel as K

        tau, v_th, v_reset, flags, _, _, samples, heads, cph, tokens, scale = spec
        bits, _, v_last = K._run_forward_packed(L.NEURON_LIF, x_seq, v_init, None, tau, v_th, v_reset, flags, False)
        out = _ssa_packed(bits, None, x_seq.dtype, samples, heads, cph, tokens, scale)
        return out, v_last, bits

    @staticmethod
    def setup_context(ctx, inputs, output):
        x_seq, v_init, spec = inputs
        ctx.spec = spec
        ctx.save_for_backward(x_seq, v_init, output[2])
        ctx.mark_non_differentiable(output[2])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_out, grad_v_last, grad_bits):
        del grad_bits
        x_seq, v_init, bits = ctx.saved_tensors
        need = bool(ctx.needs_input_grad[1])
        gx, gvi = _lif_ssa_backward(x_seq, v_init, bits, ctx.spec, grad_out, grad_v_last, need)
        return gx, (gvi if need else None), None


def _lif_ssa_backward(x_seq, v_init, bits, spec, grad_out, grad_v_last, need_gvi: bool):
    """``(grad_x_seq, grad_v_init or None)`` of ``_LifSsa``: the contraction writes the dense spike gradient from the
    bits, the LIF backward replays its forward from ``x_seq``."""
    from . import neuron_kernel as K

    tau, v_th, v_reset, flags, sg_id, sg_alpha, samples, heads, cph, tokens, scale = spec
    grad_spikes = None
    if grad_out is not None:
        grad_spikes = _ssa_packed(bits, grad_out, x_seq.dtype, samples, heads, cph, tokens, scale).view(x_seq.shape)
    gx, gvi, _ = K._run_backward(L.NEURON_LIF, grad_spikes, None, grad_v_last, None, x_seq, v_init, None, tau, v_th,
                                 v_reset, flags, sg_id, sg_alpha, need_gvi)
    return gx, (gvi if need_gvi else None)


def lif_ssa_fused(x_seq: torch.Tensor, v_init: torch.Tensor, tau: float, v_th: float, v_reset: float, flags: int,
                  sg_id: int, sg_alpha: float, heads: int, channels_per_head: int, tokens: int, scale: float
                  ) -> tuple[torch.Tensor, torch.Tensor]:
    """``x_seq`` is ``[T, N]`` with ``N = B * 3 * heads * channels_per_head * tokens``, ``v_init`` ``[N]``.  Returns
    ``(out [T*B, heads, channels_per_head, tokens], v_last [N])``.  The caller has checked ``ssa_packed_supported``,
    ``N % 8 == 0`` and that the replay backward serves the shape."""
    samples = x_seq.shape[0] * (x_seq.shape[1] // (3 * heads * channels_per_head * tokens))
    spec = (tau, v_th, v_reset, flags, sg_id, sg_alpha, samples, heads, channels_per_head, tokens, scale)
    if torch.compiler.is_compiling():  # the same launches as torch.library operators (schema, fake kernels)
        from . import fused_ops as O

        return O.lif_ssa(x_seq, v_init, spec)
    out, v_last, _ = _LifSsa.apply(x_seq, v_init, spec)
    return out, v_last
