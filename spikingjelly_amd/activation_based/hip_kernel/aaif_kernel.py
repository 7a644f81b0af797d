"""``torch.library`` operator for the activation-aware IF kernel of ``libsjhip.so``.

Counterpart of the reference's ``sj::multistep_activation_aware_if_forward``
(``triton_kernel/neuron_kernel/activation_aware_if.py:161-285``): inference only; thresholds and offsets are scalar or
one value per channel, ``channel_size`` and ``inner_size`` describe where the channel axis sits in a flattened step.
"""

from __future__ import annotations

import torch

from . import library as L
from .neuron_kernel import _state_arg

__all__ = ["hip_multistep_activation_aware_if"]


def _parameter_on_device(name: str, value: torch.Tensor, ref: torch.Tensor, channel_size: int) -> torch.Tensor:
    if value.dim() > 1 or value.numel() not in (1, channel_size):
        raise ValueError(f"{name} must be a scalar or hold one value per channel ({channel_size}), got shape "
                         f"{tuple(value.shape)}")
    return value.detach().to(device=ref.device, dtype=torch.float32).reshape(-1).contiguous()


@torch.library.custom_op("sj::hip_multistep_activation_aware_if", mutates_args=())
def hip_multistep_activation_aware_if(x_seq: torch.Tensor, v_init: torch.Tensor, v_threshold: torch.Tensor,
                                      v_offset: torch.Tensor, channel_size: int, inner_size: int, v_reset: float,
                                      soft_reset: bool, store_v_seq: bool, mode_flags: int
                                      ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``x_seq`` is ``[T, N]``, ``v_init`` ``[N]``.  Returns ``(spike_seq, v_seq, v_last)``; ``v_seq`` is an empty
    tensor unless ``store_v_seq``."""
    L.require_device_tensor("x_seq", x_seq)
    L.require_device_tensor("v_init", v_init)
    if x_seq.dim() != 2 or x_seq.shape[0] < 1 or x_seq.shape[1] < 1:
        raise ValueError(f"x_seq must be [T, N] with T, N >= 1, got shape {tuple(x_seq.shape)}")
    if v_init.shape != x_seq.shape[1:] or v_init.dtype != x_seq.dtype:
        raise ValueError(f"v_init must have shape {tuple(x_seq.shape[1:])} and dtype {x_seq.dtype}")
    dtype = L.dtype_id(x_seq.dtype)
    x_seq = x_seq.contiguous()
    T, N = x_seq.shape
    v_init, broadcast = _state_arg(v_init, False)
    threshold = _parameter_on_device("v_threshold", v_threshold, x_seq, channel_size)
    offset = _parameter_on_device("v_offset", v_offset, x_seq, channel_size)
    flags = (int(mode_flags) & L.FLAG_FP32_STATE) | broadcast | (L.FLAG_SOFT_RESET if soft_reset else 0)
    spike_seq = torch.empty_like(x_seq)
    v_seq = torch.empty_like(x_seq) if store_v_seq else x_seq.new_empty((0,))
    v_last = x_seq.new_empty((N,))
    with torch.cuda.device(x_seq.device):
        rc = L.load().sjhip_aaif_forward(
            dtype, flags, T, N, x_seq.data_ptr(), v_init.data_ptr(),
            threshold.data_ptr(), threshold.numel(), offset.data_ptr(), offset.numel(),
            int(channel_size), int(inner_size), float(v_reset),
            spike_seq.data_ptr(), v_seq.data_ptr() if store_v_seq else None, v_last.data_ptr(),
            L.current_stream_ptr(x_seq.device),
        )
    L.check(rc, "aaif_forward")
    return spike_seq, v_seq, v_last


@hip_multistep_activation_aware_if.register_fake
def _(x_seq, v_init, v_threshold, v_offset, channel_size, inner_size, v_reset, soft_reset, store_v_seq, mode_flags):
    return (x_seq.new_empty(x_seq.shape), x_seq.new_empty(x_seq.shape) if store_v_seq else x_seq.new_empty((0,)),
            v_init.new_empty(v_init.shape))
