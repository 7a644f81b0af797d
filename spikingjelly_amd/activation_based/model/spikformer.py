"""The two convolution blocks of the reference's Spikformer that sit on the fused convolution / batch-norm / LIF
path (reference ``model/spikformer.py:16-99`` ``SpikformerConv2dBN`` and ``:107-212`` ``SpikformerConv2dBNLIF``).  The
rest of that model (patch stem, MLP, classifier) is built from these two, ``SpikingSelfAttention`` and torch layers.

With ``backend='hip'`` and no pooling between batch norm and the neuron, ``SpikformerConv2dBNLIF`` runs batch norm and
the LIF fused (``layer/fused.py``); a kernel-size-1 convolution runs on the library's split-operand GEMM kernels as well, any other
convolution stays with torch and hands its output to the fused batch norm + LIF.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import base, layer, neuron
from ..layer import fused

__all__ = ["SpikformerConv2dBN", "SpikformerConv2dBNLIF"]


class SpikformerConv2dBN(nn.Module):
    def __init__(self, in_channels: int, out_channels: int, kernel_size: int, stride: int = 1, padding: int = 0,
                 pool: bool = False):
        super().__init__()
        layers = [
            nn.Conv2d(in_channels, out_channels, kernel_size=kernel_size, stride=stride, padding=padding, bias=False),
            nn.BatchNorm2d(out_channels),
        ]
        if pool:
            layers.append(nn.MaxPool2d(kernel_size=3, stride=2, padding=1))
        self.block = layer.SeqToANNContainer(*layers)

    def forward(self, x_seq: torch.Tensor):
        return self.block(x_seq)

    def __spatial_split__(self):
        return tuple(self.block.children())


class SpikformerConv2dBNLIF(nn.Module, base.MultiStepModule):
    def __init__(self, in_channels: int, out_channels: int, kernel_size: int, stride: int = 1, padding: int = 0,
                 pool: bool = False, backend: str = "torch", tau: float = 2.0, detach_reset: bool = True):
        super().__init__()
        self.conv_bn = SpikformerConv2dBN(in_channels=in_channels, out_channels=out_channels, kernel_size=kernel_size,
                                          stride=stride, padding=padding, pool=pool)
        self.neuron = neuron.LIFNode(tau=tau, detach_reset=detach_reset, step_mode="m", backend=backend)

    def forward(self, x_seq: torch.Tensor):
        block = self.conv_bn.block
        if (self.neuron.backend == "hip" and len(block) == 2 and x_seq.dim() == 5
                and fused.unobserved(self.conv_bn, block, block[0], block[1], self.neuron)):
            conv, bn = block[0], block[1]
            out = fused.conv_bn_lif(x_seq, conv, bn, self.neuron)
            if out is None:
                y = conv(x_seq.flatten(0, 1))
                out = fused.conv_bn_lif(y.view(x_seq.shape[0], x_seq.shape[1], *y.shape[1:]), None, bn, self.neuron)
                if out is None:
                    out = self.neuron(bn(y).view(x_seq.shape[0], x_seq.shape[1], *y.shape[1:]))
            return out
        return self.neuron(self.conv_bn(x_seq))

    def __spatial_split__(self):
        return self.conv_bn, self.neuron
