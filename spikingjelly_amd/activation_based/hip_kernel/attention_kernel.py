"""``torch.library`` operators for the spiking self-attention contraction on the matrix cores.

    sj::hip_ssa_forward(qkv [S, 3, H, Cph, L], scale)            -> out [S, H, Cph, L]
    sj::hip_ssa_backward(qkv, grad_out, scale)                    -> grad_qkv

``out = scale * (v @ k^T) @ q`` per (sample, head), the contraction of the reference's
``SpikingSelfAttention._ssa_kernel_torch`` (layer/attention.py:346-353).  qkv must hold binary spikes.
"""

from __future__ import annotations

import torch

from . import library as L

__all__ = ["hip_ssa_forward", "hip_ssa_backward", "ssa_supported"]


def ssa_supported(dtype: torch.dtype, channels_per_head: int, tokens: int) -> bool:
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
