"""Spike compressors used by input-compressed gradient checkpointing.

Counterpart of the reference's ``memopt/compress.py`` (:57-166 base class, :168-221 Null, :223-275
Boolean, :278-329 Uint8, :332-385 Bit).  ``BitSpikeCompressor`` packs 8 binary spikes per byte: tensors on a
ROCm device go through the HIP kernels (``hip_kernel/compress.py``, no other path), tensors on the CPU through
the torch ops below, which restate the reference's torch path for non-CUDA tensors
(``triton_kernel/compress.py:19-44``) and give the same bytes.
"""

from __future__ import annotations

import abc

import torch

from ..hip_kernel import compress as _hip

__all__ = [
    "BaseSpikeCompressor",
    "NullSpikeCompressor",
    "BooleanSpikeCompressor",
    "Uint8SpikeCompressor",
    "BitSpikeCompressor",
    "bit_spike_compress",
    "bit_spike_decompress",
]


def _torch_bit_spike_compress(s_seq: torch.Tensor) -> torch.Tensor:
    bits = s_seq.to(dtype=torch.bool).reshape(-1)
    n_bytes = (bits.numel() + 7) // 8
    packed = torch.zeros(n_bytes, dtype=torch.uint8, device=bits.device)
    for i in range(8):
        lane = bits[i::8].to(torch.uint8)
        if lane.numel() > 0:
            packed[: lane.numel()] |= lane << i
    return packed


def _torch_bit_spike_decompress(packed: torch.Tensor, shape, dtype: torch.dtype) -> torch.Tensor:
    n = torch.Size(shape).numel()
    out = torch.zeros(n, dtype=torch.uint8, device=packed.device)
    for i in range(8):
        count = (n - i + 7) // 8
        out[i::8] = ((packed >> i) & 1)[:count]
    return out.reshape(shape).to(dtype)


def bit_spike_compress(s_seq: torch.Tensor) -> torch.Tensor:
    """Device dispatch of the reference's ``bit_spike_compress`` (triton_kernel/compress.py:114-166)."""
    if s_seq.device.type == "cuda":
        return _hip.bit_spike_compress(s_seq)
    return _torch_bit_spike_compress(s_seq)


def bit_spike_decompress(s_seq_compressed: torch.Tensor, shape, dtype: torch.dtype = torch.uint8) -> torch.Tensor:
    """Device dispatch of the reference's ``bit_spike_decompress`` (triton_kernel/compress.py:169-221)."""
    if s_seq_compressed.device.type == "cuda":
        return _hip.bit_spike_decompress(s_seq_compressed, shape, dtype)
    return _torch_bit_spike_decompress(s_seq_compressed, torch.Size(shape), dtype)


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
