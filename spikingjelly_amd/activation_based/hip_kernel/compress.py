"""Spike bit-packing on the device: 8 binary spikes per byte, LSB first over the flattened tensor.

Counterpart of the device kernels of the reference's ``triton_kernel/compress.py:114-221``
(``bit_spike_compress`` / ``bit_spike_decompress``).  These functions run ``libsjhip.so`` on ROCm tensors only
and raise for anything else; the torch path the reference keeps for non-CUDA tensors (compress.py:19-44,
150-151) lives with the compressor classes in ``memopt/compress.py``.
"""

from __future__ import annotations

import torch

from . import library as L

__all__ = ["bit_spike_compress", "bit_spike_decompress"]


def bit_spike_compress(s_seq: torch.Tensor) -> torch.Tensor:
    """Pack a strictly binary tensor into ``(numel + 7) // 8`` bytes (uint8, 1-D)."""
    L.require_device_tensor("s_seq", s_seq)
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
    L.require_device_tensor("s_seq_compressed", s_seq_compressed)
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
