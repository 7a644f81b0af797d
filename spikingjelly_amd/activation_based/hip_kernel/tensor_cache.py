"""Binary spikes kept for a backward pass as ``bool`` or as bits.

Counterpart of the reference's ``cuda_kernel/tensor_cache.py``: ``float_spike_to_bool`` (:95-187),
``bool_spike_to_float`` (:190-283), ``tensor_key`` (:286-288), ``BoolTensorCache`` (:291-330) and the process-wide
``BOOL_TENSOR_CACHE`` (:333).  The byte layout is the one of the reference's ``float2bool`` / ``bool2float`` kernels
(:16-93): byte ``j`` bit ``i`` is element ``8 j + i`` of the flattened tensor, the tail padded with zero bits.  That is
also the layout of ``bit_spike_compress``, so tensors on a ROCm device go through the same two HIP kernels
(``sjhip_bit_pack`` / ``sjhip_bit_unpack``, no other path for them); CPU tensors take the torch ops the reference
uses when CuPy is absent (:173-176, 270-274).
"""

from __future__ import annotations

import threading
from typing import Union

import torch

from ... import configure
from . import compress

__all__ = ["float_spike_to_bool", "bool_spike_to_float", "tensor_key", "BoolTensorCache", "BOOL_TENSOR_CACHE"]

_SPIKE_DTYPES = (torch.float32, torch.float16)


def float_spike_to_bool(spike: torch.Tensor):
    """``(spike_b, s_dtype, s_shape, s_padding)``: ``spike`` (float32 or float16, every element 0 or 1) packed eight
    to a byte.  ``s_padding = 8 - numel % 8`` is the reference's count of pad elements, 8 meaning none."""
    if spike.dtype not in _SPIKE_DTYPES:
        raise NotImplementedError(spike.dtype)
    s_dtype, s_shape = spike.dtype, spike.shape
    flat = spike.flatten()
    s_padding = 8 - flat.numel() % 8
    if flat.is_cuda:
        return compress.bit_spike_compress(flat), s_dtype, s_shape, s_padding
    if s_padding != 8:
        flat = torch.nn.functional.pad(flat, (0, s_padding))
    lanes = flat.view(-1, 8).to(torch.uint8)
    spike_b = torch.zeros(lanes.shape[0], dtype=torch.uint8, device=flat.device)
    for i in range(8):
        spike_b += lanes[:, i] << i
    return spike_b, s_dtype, s_shape, s_padding


def bool_spike_to_float(spike_b: torch.Tensor, s_dtype: torch.dtype, s_shape: torch.Size, s_padding: int = 0):
    """Inverse of :func:`float_spike_to_bool`: the 0/1 tensor of ``s_dtype`` and ``s_shape``."""
    if s_dtype not in _SPIKE_DTYPES:
        raise NotImplementedError(s_dtype)
    padded = spike_b.numel() * 8
    n = padded - s_padding if s_padding not in (0, 8) else padded
    if spike_b.is_cuda:
        return compress.bit_spike_decompress(spike_b, (n,), s_dtype).reshape(s_shape)
    lanes = torch.zeros((spike_b.numel(), 8), dtype=s_dtype, device=spike_b.device)
    for i in range(8):
        lanes[:, i] = (spike_b >> i) & 1
    return lanes.flatten()[:n].reshape(s_shape)


def tensor_key(x: torch.Tensor):
    """``(address of the first element, address of the last element, numel)``: what identifies the tensor a forward
    stored until its backward fetches it.  Equal to the reference's key for a contiguous tensor; computed from the
    strides, without the temporary copy the reference's ``flatten()`` makes of a non-contiguous one."""
    last = sum((size - 1) * stride for size, stride in zip(x.shape, x.stride())) if x.numel() else 0
    return x.data_ptr(), x.data_ptr() + last * x.element_size(), x.numel()


class BoolTensorCache:
    """Spikes stored once per tensor, however many operators consume it (reference counted, thread-safe)."""

    def __init__(self):
        self.cache = {}
        self.lock = threading.Lock()

    def store_bool(self, spike: Union[torch.FloatTensor, torch.HalfTensor]):
        key = tensor_key(spike)
        with self.lock:
            entry = self.cache.get(key)
            if entry is not None:
                payload, users = entry
                self.cache[key] = payload, users + 1
                return key
            level = configure.save_bool_spike_level
            if level == 0:
                payload = (0, spike.bool(), spike.dtype)
            elif level == 1:
                payload = (1,) + tuple(float_spike_to_bool(spike))
            else:
                raise NotImplementedError(f"save_bool_spike_level={level}")
            self.cache[key] = payload, 1
        return key

    def get_float(self, tk, spike_shape: torch.Size):
        with self.lock:
            payload, users = self.cache[tk]
            if users == 1:
                del self.cache[tk]
            else:
                self.cache[tk] = payload, users - 1
        # the form is the one chosen when the tensor was stored, whatever the switch says now
        if payload[0] == 0:
            return payload[1].to(payload[2]).view(spike_shape)
        return bool_spike_to_float(*payload[1:]).view(spike_shape)


BOOL_TENSOR_CACHE = BoolTensorCache()
