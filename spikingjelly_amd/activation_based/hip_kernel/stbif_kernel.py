"""``torch.library`` operator for the ST-BIF kernel of ``libsjhip.so`` (SpikeZIP's signed ternary neuron).

Counterpart of the reference's ``sj::multi_step_stbif`` / ``sj::single_step_stbif``
(``triton_kernel/neuron_kernel/stbif.py:258-416``): inference only, returns the output sequence, the three states
after the last step and an int32 work flag (non-zero when any input or output of the call was non-zero).  The
quantiser scale and the accumulator bounds are tensors, as in the reference; they are read on the device, so no
``.item()`` synchronisation happens here.
"""

from __future__ import annotations

import torch

from . import library as L
from .neuron_kernel import _state_arg

__all__ = ["hip_multistep_stbif"]


def _scalar_on_device(name: str, value: torch.Tensor, ref: torch.Tensor) -> torch.Tensor:
    if value.numel() != 1:
        raise ValueError(f"{name} must hold one element, got shape {tuple(value.shape)}")
    return value.detach().to(device=ref.device, dtype=torch.float32).reshape(1).contiguous()


@torch.library.custom_op("sj::hip_multistep_stbif", mutates_args=())
def hip_multistep_stbif(x_seq: torch.Tensor, q: torch.Tensor, acc_q: torch.Tensor, q_threshold: torch.Tensor,
                        pos_max: torch.Tensor, neg_min: torch.Tensor, mode_flags: int
                        ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``x_seq`` is ``[T, N]``, ``q`` and ``acc_q`` are ``[N]`` (an expanded one-element tensor is read as one
    element).  Returns ``(out_seq, q_final, acc_q_final, cur_output, work_flag)``."""
    L.require_device_tensor("x_seq", x_seq)
    L.require_device_tensor("q", q)
    L.require_device_tensor("acc_q", acc_q)
    if x_seq.dim() != 2 or x_seq.shape[0] < 1 or x_seq.shape[1] < 1:
        raise ValueError(f"x_seq must be [T, N] with T, N >= 1, got shape {tuple(x_seq.shape)}")
    for name, state in (("q", q), ("acc_q", acc_q)):
        if state.shape != x_seq.shape[1:] or state.dtype != x_seq.dtype:
            raise ValueError(f"{name} must have shape {tuple(x_seq.shape[1:])} and dtype {x_seq.dtype}, got "
                             f"{tuple(state.shape)} {state.dtype}")
    dtype = L.dtype_id(x_seq.dtype)
    x_seq = x_seq.contiguous()
    T, N = x_seq.shape
    q, q_flag = _state_arg(q, False)
    acc_q, acc_flag = _state_arg(acc_q, False)
    flags = int(mode_flags) & L.FLAG_FP32_STATE
    if q_flag:
        flags |= L.FLAG_Q_BROADCAST
    if acc_flag:
        flags |= L.FLAG_ACC_BROADCAST
    scalars = [_scalar_on_device(n, v, x_seq) for n, v in
               (("q_threshold", q_threshold), ("pos_max", pos_max), ("neg_min", neg_min))]
    out_seq = torch.empty_like(x_seq)
    q_final, acc_final, cur = x_seq.new_empty((N,)), x_seq.new_empty((N,)), x_seq.new_empty((N,))
    work = torch.zeros((), dtype=torch.int32, device=x_seq.device)
    with torch.cuda.device(x_seq.device):
        rc = L.load().sjhip_stbif_forward(
            dtype, flags, T, N, x_seq.data_ptr(), q.data_ptr(), acc_q.data_ptr(),
            scalars[0].data_ptr(), scalars[1].data_ptr(), scalars[2].data_ptr(),
            out_seq.data_ptr(), q_final.data_ptr(), acc_final.data_ptr(), cur.data_ptr(), work.data_ptr(),
            L.current_stream_ptr(x_seq.device),
        )
    L.check(rc, "stbif_forward")
    return out_seq, q_final, acc_final, cur, work


@hip_multistep_stbif.register_fake
def _(x_seq, q, acc_q, q_threshold, pos_max, neg_min, mode_flags):
    n = x_seq.shape[1:]
    return (x_seq.new_empty(x_seq.shape), x_seq.new_empty(n), x_seq.new_empty(n), x_seq.new_empty(n),
            x_seq.new_empty((), dtype=torch.int32))
