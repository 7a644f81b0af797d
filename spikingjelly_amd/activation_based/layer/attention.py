"""Spikformer-style spiking self-attention (reference ``layer/attention.py:245-387``).

``Conv1d+BN -> LIF -> scale * (V K^T) Q -> LIF(v_threshold=0.5) -> Conv1d+BN -> LIF`` on ``[T, N, C, L]``
input.  With ``backend='hip'`` the three LIF nodes run the HIP neuron kernels and the contraction runs on
the matrix cores (int8 / bf16 MFMA, fp32 accumulation; exact because Q/K/V are binary).  For fp32 device tensors whose
token count is a multiple of 4 the two ``Conv1d(k=1) -> BatchNorm1d -> LIF`` chains run fused as well (``layer/fused.py``:
split-bf16 MFMA GEMMs, batch norm and the neuron in two passes over the convolution output); other inputs keep
torch's convolution and batch norm around the hip neurons.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from ... import configure
from .. import base, neuron
from . import fused
from .container import SeqToANNContainer


class SpikingSelfAttention(nn.Module, base.MultiStepModule):
    def __init__(self, dim, num_heads=8, backend: str = "torch"):
        super().__init__()
        if dim % num_heads != 0:
            raise ValueError(f"dim {dim} should be divided by num_heads {num_heads}.")
        self.dim = dim
        self.num_heads = num_heads
        self.head_dim = dim // num_heads
        self.scale = 0.125
        self.qkv_conv_bn = SeqToANNContainer(
            nn.Conv1d(dim, dim * 3, kernel_size=1, stride=1, bias=False),
            nn.BatchNorm1d(dim * 3),
        )
        self.qkv_lif = neuron.LIFNode(tau=2.0, detach_reset=True, step_mode="m", backend=backend)
        self.attn_lif = neuron.LIFNode(tau=2.0, v_threshold=0.5, detach_reset=True, step_mode="m", backend=backend)
        self.proj_conv_bn = SeqToANNContainer(
            nn.Conv1d(dim, dim, kernel_size=1, stride=1, bias=False),
            nn.BatchNorm1d(dim),
        )
        self.proj_lif = neuron.LIFNode(tau=2.0, detach_reset=True, step_mode="m", backend=backend)

    @property
    def backend(self):
        return self.qkv_lif.backend

    @backend.setter
    def backend(self, value: str):
        self.qkv_lif.backend = value
        self.attn_lif.backend = value
        self.proj_lif.backend = value

    @property
    def supported_backends(self):
        return self.qkv_lif.supported_backends

    @staticmethod
    def _ssa_kernel_torch(qkv, scale):
        # qkv [T, N, 3, heads, Cph, L] -> [T, N, heads, Cph, L]
        qt, kt, vt = qkv.flatten(2, 3).chunk(3, dim=2)
        x_seq = vt @ kt.transpose(-2, -1)
        return (x_seq @ qt) * scale

    @staticmethod
    def _ssa_kernel_hip(qkv, scale):
        from ..hip_kernel.attention_kernel import hip_ssa_forward

        T, N = qkv.shape[:2]
        out = hip_ssa_forward(qkv.flatten(0, 1), scale)
        return out.view(T, N, *out.shape[1:])

    def _lif_ssa_fused(self, pre: torch.Tensor):
        """``qkv_lif`` and the contraction as one step whose spikes exist only bit-packed (1/32 of the fp32 spike
        tensor: the LIF writes bits, the contraction reads bits, the backward keeps bits).  Returns ``None`` when the
        shape, the mode or the state does not allow it; the two-operator path then runs.  Results are identical."""
        from ..functional import neuron as F
        from ..hip_kernel import attention_kernel as A
        from ..hip_kernel import neuron_kernel as K
        from ..hip_kernel.surrogate_registry import resolve_sg_hip_id_and_alpha

        node = self.qkv_lif
        T, N, C3, L = pre.shape
        cph = C3 // 3 // self.num_heads
        if (not fused._plain_hip_lif(node) or not fused.unobserved(node) or not pre.is_cuda
                or not A.ssa_packed_supported(pre.dtype, cph, L) or (N * C3 * L) % 8 != 0):
            return None
        x2 = pre.flatten(1)
        need_grad = torch.is_grad_enabled() and pre.requires_grad
        if need_grad and not F._hip_recompute(x2):
            return None  # the fused backward replays the LIF forward
        node._check_hip_surrogate()
        (v,) = node.materialize_states((pre,), (node.v,), "m")
        if need_grad and v.requires_grad:
            return None
        soft = node.v_reset is None
        flags = K._flags(soft, node.detach_reset, node.decay_input, F._hip_mode_flags(pre))
        sg_id, sg_alpha = resolve_sg_hip_id_and_alpha(node.surrogate_function) if need_grad else (0, 0.0)
        with torch.set_grad_enabled(need_grad):
            out, v_last = A.lif_ssa_fused(x2, v.flatten(), float(node.tau), node.v_threshold, 0.0 if soft else float(node.v_reset),
                                          flags, sg_id, sg_alpha, self.num_heads, cph, L, self.scale)
        node.v = v_last.reshape(pre.shape[1:])
        return out.view(T, N, self.num_heads, cph, L)

    def forward(self, x_seq: torch.Tensor):
        if x_seq.ndim != 4:
            raise ValueError(f"expected 4D input with shape [T, N, C, L], but got input with shape {x_seq.shape}")
        T, N, C, L = x_seq.shape
        hip = self.backend == "hip"
        out = None
        attn_spikes = None
        if hip and len(self.qkv_conv_bn) == 2:
            # convolution, batch norm, LIF (bit-packed spikes), the contraction and the attention's LIF in one autograd
            # node; without the last of them when it cannot run inside the contraction
            if configure.hip_fuse_ssa_lif:
                attn_spikes = fused.conv_bn_lif(x_seq, self.qkv_conv_bn[0], self.qkv_conv_bn[1], self.qkv_lif,
                                                ssa=(self.num_heads, self.scale), attn=self.attn_lif,
                                                container=self.qkv_conv_bn)
            if attn_spikes is None:
                out = fused.conv_bn_lif(x_seq, self.qkv_conv_bn[0], self.qkv_conv_bn[1], self.qkv_lif,
                                        ssa=(self.num_heads, self.scale), container=self.qkv_conv_bn)
        if out is None and attn_spikes is None:
            pre = self.qkv_conv_bn(x_seq)  # [T, N, 3*C, L]
            local_dim = pre.shape[2] // 3
            if local_dim % self.num_heads != 0:
                raise ValueError(f"local qkv dim {local_dim} is not divisible by num_heads={self.num_heads}.")
            out = self._lif_ssa_fused(pre) if hip else None
            if out is None:
                qkv = self.qkv_lif(pre).reshape(T, N, 3, self.num_heads, local_dim // self.num_heads, L)
                out = self._ssa_kernel_hip(qkv, self.scale) if hip else self._ssa_kernel_torch(qkv, self.scale)
        y = None
        if attn_spikes is None and hip and len(self.proj_conv_bn) == 2:
            # the attention's LIF writes its spikes as bits, the projection's convolution reads bits
            y = fused.lif_conv_bn_lif(out, self.attn_lif, self.proj_conv_bn[0], self.proj_conv_bn[1], self.proj_lif,
                                      container=self.proj_conv_bn)
            if y is not None:
                return y
        if attn_spikes is None:
            attn_spikes = self.attn_lif(out)
        local_dim = attn_spikes.shape[2] * attn_spikes.shape[3]
        x_seq = attn_spikes.reshape(T, N, local_dim, L)
        if hip and len(self.proj_conv_bn) == 2:
            y = fused.conv_bn_lif(x_seq, self.proj_conv_bn[0], self.proj_conv_bn[1], self.proj_lif, x_exact=True,
                                  container=self.proj_conv_bn)
        if y is None:
            y = self.proj_lif(self.proj_conv_bn(x_seq))
        return y  # [T, N, C, L]

    def extra_repr(self):
        return f"dim={self.dim}, num_heads={self.num_heads}, backend={self.backend}"
