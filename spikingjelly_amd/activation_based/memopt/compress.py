"""Spike compressors used by input-compressed gradient checkpointing.

Counterpart of the reference's ``memopt/compress.py`` (:57-166 base class, :168-221 Null, :223-275
Boolean, :278-329 Uint8, :332-385 Bit).  ``BitSpikeCompressor`` packs 8 binary spikes per byte through
the HIP kernels for device tensors; CPU tensors use the torch path with the same byte layout.
"""

from __future__ import annotations

import abc

import torch

from ..hip_kernel.compress import bit_spike_compress, bit_spike_decompress

__all__ = [
    "BaseSpikeCompressor",
    "NullSpikeCompressor",
    "BooleanSpikeCompressor",
    "Uint8SpikeCompressor",
    "BitSpikeCompressor",
]


class BaseSpikeCompressor(abc.ABC):
    """``compress`` / ``decompress`` run under ``no_grad``; subclasses implement the ``_`` versions."""

    requires_strictly_binary = False

    @abc.abstractmethod
    def _compress(self, s_seq: torch.Tensor) -> torch.Tensor:
        ...

    @abc.abstractmethod
    def _decompress(self, s_seq: torch.Tensor, shape) -> torch.Tensor:
        ...

    def compress(self, s_seq: torch.Tensor) -> torch.Tensor:
        with torch.no_grad():
            return self._compress(s_seq)

    def decompress(self, s_seq: torch.Tensor, shape) -> torch.Tensor:
        with torch.no_grad():
            return self._decompress(s_seq, shape)


class NullSpikeCompressor(BaseSpikeCompressor):
    def _compress(self, s_seq):
        return s_seq

    def _decompress(self, s_seq, shape):
        return s_seq


class BooleanSpikeCompressor(BaseSpikeCompressor):
    requires_strictly_binary = True

    def __init__(self):
        self.s_seq_dtype = torch.float32

    def _compress(self, s_seq):
        self.s_seq_dtype = s_seq.dtype
        return s_seq.to(torch.bool)

    def _decompress(self, s_seq, shape):
        return s_seq.to(dtype=self.s_seq_dtype).reshape(shape)


class Uint8SpikeCompressor(BaseSpikeCompressor):
    def __init__(self):
        self.s_seq_dtype = torch.float32

    def _compress(self, s_seq):
        self.s_seq_dtype = s_seq.dtype
        return s_seq.to(torch.uint8)

    def _decompress(self, s_seq, shape):
        return s_seq.to(dtype=self.s_seq_dtype).reshape(shape)


class BitSpikeCompressor(BaseSpikeCompressor):
    """8 spikes per byte, LSB first over the flattened tensor; input must be strictly 0/1.

    Decompression returns ``float32`` whatever the input dtype was, as the reference does (its
    ``_compress`` never records the input dtype, memopt/compress.py:376-385).
    """

    requires_strictly_binary = True

    def __init__(self):
        self.s_seq_dtype = torch.float32

    def _compress(self, s_seq):
        return bit_spike_compress(s_seq)

    def _decompress(self, s_seq, shape):
        return bit_spike_decompress(s_seq, shape, dtype=self.s_seq_dtype)
