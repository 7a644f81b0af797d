"""Linear and convolution layers whose input is a binary spike tensor, kept for the backward as bool or bits.

Counterpart of the reference's ``cuda_kernel/spike_op.py`` (operators :124-257, functions :291-520, layers :523-734).
The arithmetic is torch's own ``F.linear`` / ``F.conv*``; what the operators change is what autograd holds between
forward and backward: not the float spike tensor but its entry in ``tensor_cache.BOOL_TENSOR_CACHE`` (one byte per
spike, or one bit with ``configure.save_bool_spike_level = 1``, packed and unpacked by this library's HIP kernels).
The convolution backward is ATen's ``convolution_backward`` called directly; the reference compiles a C++ shim at
import time to reach the same routine (:34-59).

CPU tensors, and string paddings, run the plain torch function, as in the reference (:331-334, 389-392).
"""

from __future__ import annotations

from typing import Optional, Union

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.nn.modules.utils import _pair, _single, _triple

from . import tensor_cache

__all__ = ["spike_linear", "spike_conv1d", "spike_conv2d", "spike_conv3d", "SpikeLinear", "SpikeConv1d",
           "SpikeConv2d", "SpikeConv3d", "hip_spike_linear_forward", "hip_spike_convolution_forward"]

_CONVS = {3: (F.conv1d, _single), 4: (F.conv2d, _pair), 5: (F.conv3d, _triple)}


def _conv_of(spike: torch.Tensor):
    if spike.dim() not in _CONVS:
        raise ValueError(f"spikeConvolution only supports 3D/4D/5D input, but got dim={spike.dim()}.")
    return _CONVS[spike.dim()]


@torch.library.custom_op("sj::hip_spike_linear_forward", mutates_args=())
def hip_spike_linear_forward(spike: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    return F.linear(spike, weight, bias)


@hip_spike_linear_forward.register_fake
def _(spike, weight, bias):
    return spike.new_empty(spike.shape[:-1] + (weight.shape[0],))


def _linear_setup(ctx, inputs, output):
    spike, weight, bias = inputs
    ctx.s_shape = spike.shape
    ctx.s_tk = tensor_cache.BOOL_TENSOR_CACHE.store_bool(spike)
    ctx.save_for_backward(weight)
    ctx.has_bias = bias is not None


def _linear_backward(ctx, grad_output):
    (weight,) = ctx.saved_tensors
    spike = tensor_cache.BOOL_TENSOR_CACHE.get_float(ctx.s_tk, ctx.s_shape)
    rows = grad_output.reshape(-1, grad_output.shape[-1])
    grad_spike = F.linear(grad_output, weight.to(grad_output.dtype).t())
    grad_weight = torch.mm(rows.t(), spike.reshape(-1, spike.shape[-1]).to(grad_output.dtype))
    return grad_spike, grad_weight, (rows.sum(0) if ctx.has_bias else None)


torch.library.register_autograd("sj::hip_spike_linear_forward", _linear_backward, setup_context=_linear_setup)


@torch.library.custom_op("sj::hip_spike_convolution_forward", mutates_args=())
def hip_spike_convolution_forward(spike: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                                  stride: list[int], padding: list[int], dilation: list[int], groups: int
                                  ) -> torch.Tensor:
    conv, _ = _conv_of(spike)
    return conv(spike, weight, bias, stride, padding, dilation, groups)


@hip_spike_convolution_forward.register_fake
def _(spike, weight, bias, stride, padding, dilation, groups):
    conv, _ = _conv_of(spike)
    return conv(spike, weight, bias, stride, padding, dilation, groups)


def _conv_setup(ctx, inputs, output):
    spike, weight, bias, stride, padding, dilation, groups = inputs
    _, ntuple = _conv_of(spike)
    ctx.geometry = (list(ntuple(stride)), list(ntuple(padding)), list(ntuple(dilation)), groups)
    ctx.wants = (bool(spike.requires_grad), bool(weight.requires_grad), bool(bias is not None and bias.requires_grad))
    ctx.save_for_backward(weight)
    ctx.s_shape, ctx.s_tk = None, None
    if ctx.wants[0] or ctx.wants[1]:
        ctx.s_shape = spike.shape
        ctx.s_tk = tensor_cache.BOOL_TENSOR_CACHE.store_bool(spike)


def _conv_backward(ctx, grad_output):
    grad_spike = grad_weight = grad_bias = None
    if ctx.wants[0] or ctx.wants[1]:
        (weight,) = ctx.saved_tensors
        spike = tensor_cache.BOOL_TENSOR_CACHE.get_float(ctx.s_tk, ctx.s_shape).to(grad_output.dtype)
        stride, padding, dilation, groups = ctx.geometry
        grad_spike, grad_weight, _ = torch.ops.aten.convolution_backward(
            grad_output, spike, weight.to(grad_output.dtype), None, stride, padding, dilation, False,
            [0] * len(stride), groups, [ctx.wants[0], ctx.wants[1], False])
    if ctx.wants[2]:
        grad_bias = grad_output.sum(dim=(0, *range(2, grad_output.dim())))
    return grad_spike, grad_weight, grad_bias, None, None, None, None


torch.library.register_autograd("sj::hip_spike_convolution_forward", _conv_backward, setup_context=_conv_setup)


def spike_linear(spike: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``F.linear`` for a 0/1 ``spike``; on a GPU the backward keeps ``spike`` as bool or bits, not as floats."""
    if not spike.is_cuda:
        return F.linear(spike, weight, bias)
    return hip_spike_linear_forward(spike, weight, bias)


def _spike_conv(dim: int, spike, weight, bias, stride, padding, dilation, groups):
    conv, ntuple = _CONVS[dim]
    if not spike.is_cuda or isinstance(padding, str):
        return conv(spike, weight, bias, stride, padding, dilation, groups)
    return hip_spike_convolution_forward(spike, weight, bias, list(ntuple(stride)), list(ntuple(padding)),
                                         list(ntuple(dilation)), groups)


def spike_conv1d(spike: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 stride: Union[int, tuple] = 1, padding: Union[str, int, tuple] = "valid",
                 dilation: Union[int, tuple] = 1, groups: int = 1) -> torch.Tensor:
    """``F.conv1d`` for a 0/1 ``spike`` ``[N, C, L]``; see :func:`spike_linear`."""
    return _spike_conv(3, spike, weight, bias, stride, padding, dilation, groups)


def spike_conv2d(spike: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 stride: Union[int, tuple] = 1, padding: Union[str, int, tuple] = "valid",
                 dilation: Union[int, tuple] = 1, groups: int = 1) -> torch.Tensor:
    """``F.conv2d`` for a 0/1 ``spike`` ``[N, C, H, W]``; see :func:`spike_linear`."""
    return _spike_conv(4, spike, weight, bias, stride, padding, dilation, groups)


def spike_conv3d(spike: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 stride: Union[int, tuple] = 1, padding: Union[str, int, tuple] = "valid",
                 dilation: Union[int, tuple] = 1, groups: int = 1) -> torch.Tensor:
    """``F.conv3d`` for a 0/1 ``spike`` ``[N, C, D, H, W]``; see :func:`spike_linear`."""
    return _spike_conv(5, spike, weight, bias, stride, padding, dilation, groups)


class SpikeLinear(nn.Linear):
    """``nn.Linear`` whose input is a 0/1 spike tensor (less memory held for the backward on a GPU)."""

    def forward(self, spike: torch.Tensor) -> torch.Tensor:
        return spike_linear(spike, self.weight, self.bias)


class _SpikeConvMixin:
    _spike_conv = None
    _zero = None

    def _conv_forward(self, spike: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]):
        fn = type(self)._spike_conv
        if self.padding_mode != "zeros":
            padded = F.pad(spike, self._reversed_padding_repeated_twice, mode=self.padding_mode)
            return fn(padded, weight, bias, self.stride, type(self)._zero, self.dilation, self.groups)
        return fn(spike, weight, bias, self.stride, self.padding, self.dilation, self.groups)


class SpikeConv1d(_SpikeConvMixin, nn.Conv1d):
    """``nn.Conv1d`` whose input is a 0/1 spike tensor."""
    _spike_conv, _zero = staticmethod(spike_conv1d), _single(0)


class SpikeConv2d(_SpikeConvMixin, nn.Conv2d):
    """``nn.Conv2d`` whose input is a 0/1 spike tensor."""
    _spike_conv, _zero = staticmethod(spike_conv2d), _pair(0)


class SpikeConv3d(_SpikeConvMixin, nn.Conv3d):
    """``nn.Conv3d`` whose input is a 0/1 spike tensor."""
    _spike_conv, _zero = staticmethod(spike_conv3d), _triple(0)
