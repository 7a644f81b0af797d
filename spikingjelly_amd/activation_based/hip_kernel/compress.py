"""Spike bit-packing on the device: 8 binary spikes per byte, LSB first over the flattened tensor.

Counterpart of the reference's ``triton_kernel/compress.py:114-221`` (``bit_spike_compress`` /
``bit_spike_decompress``).  Device tensors go through ``libsjhip.so``; CPU tensors take a torch
path with the same layout, as the reference does for non-CUDA tensors (compress.py:150-151).
"""

from __future__ import annotations

import torch

from . import library as L

__all__ = ["bit_spike_compress", "bit_spike_decompress"]


def _compress_cpu(s_seq: torch.Tensor) -> torch.Tensor:
    bits = s_seq.to(dtype=torch.bool).reshape(-1)
    n_bytes = (bits.numel() + 7) // 8
    packed = torch.zeros(n_bytes, dtype=torch.uint8, device=bits.device)
    for i in range(8):
        lane = bits[i::8].to(torch.uint8)
        if lane.numel() > 0:
            packed[: lane.numel()] |= lane << i
    return packed


def _decompress_cpu(packed: torch.Tensor, shape, dtype: torch.dtype) -> torch.Tensor:
    n = torch.Size(shape).numel()
    out = torch.zeros(n, dtype=torch.uint8, device=packed.device)
    for i in range(8):
        count = (n - i + 7) // 8
        out[i::8] = ((packed >> i) & 1)[:count]
    return out.reshape(shape).to(dtype)


def bit_spike_compress(s_seq: torch.Tensor) -> torch.Tensor:
    """Pack a strictly binary tensor into ``(numel + 7) // 8`` bytes (uint8, 1-D)."""
    if s_seq.device.type != "cuda":
        return _compress_cpu(s_seq)
    src = s_seq.contiguous().reshape(-1)
    n = src.numel()
    packed = torch.empty((n + 7) // 8, dtype=torch.uint8, device=src.device)
    if n == 0:
        return packed
    with torch.cuda.device(src.device):
        rc = L.load().sjhip_bit_pack(L.dtype_id(src.dtype, allow_u8=True), n, src.data_ptr(),
                                     packed.data_ptr(), L.current_stream_ptr(src.device))
    L.check(rc, "bit_pack")
    return packed


def bit_spike_decompress(s_seq_compressed: torch.Tensor, shape, dtype: torch.dtype = torch.uint8) -> torch.Tensor:
    """Unpack to a 0/1 tensor of ``shape``.  ``dtype`` defaults to ``uint8`` like the reference's
    device kernel; passing the final dtype saves the separate cast pass."""
    shape = torch.Size(shape)
    if s_seq_compressed.device.type != "cuda":
        return _decompress_cpu(s_seq_compressed, shape, dtype)
    n = shape.numel()
    src = s_seq_compressed.contiguous()
    if src.dtype != torch.uint8 or src.numel() < (n + 7) // 8:
        raise ValueError(f"compressed tensor must be uint8 with at least {(n + 7) // 8} bytes")
    out = torch.empty(n, dtype=dtype, device=src.device)
    if n > 0:
        with torch.cuda.device(src.device):
            rc = L.load().sjhip_bit_unpack(L.dtype_id(dtype, allow_u8=True), n, src.data_ptr(),
                                           out.data_ptr(), L.current_stream_ptr(src.device))
        L.check(rc, "bit_unpack")
    return out.reshape(shape)
