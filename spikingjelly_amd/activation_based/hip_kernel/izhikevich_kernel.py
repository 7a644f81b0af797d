"""``torch.library`` operators for the Izhikevich kernels of ``libsjhip.so``.

Counterpart of the reference's ``sj::cupy_multistep_izhikevich_forward`` / ``_backward``
(``cuda_kernel/neuron_kernel/multi_step/izhikevich.py``): two states ``v`` and ``w``.

    sj::hip_multistep_izhikevich_forward  -> (spike_seq, v_seq, w_seq, v_last, w_last, h_seq)
    sj::hip_multistep_izhikevich_backward -> (grad_x_seq, grad_v_init, grad_w_init)
    sj::hip_multistep_izhikevich_backward_replay -> the same from (x_seq, v_init, w_init) instead of h_seq

``v_seq`` / ``w_seq`` are empty tensors unless ``store_v_seq`` / ``store_w_seq``; ``h_seq`` is empty unless ``save_h``
(training without ``replay``).  With ``replay`` the forward keeps no ``h_seq`` and the backward kernel recomputes it
from the inputs (no counterpart in the reference, whose kernel always saves ``h_seq``).
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import library as L
from .neuron_kernel import _state_arg

__all__ = ["hip_multistep_izhikevich_forward", "hip_multistep_izhikevich_backward",
           "hip_multistep_izhikevich_backward_replay"]


def _params(scalars: list[float], sg_id: int, sg_alpha: float, flags: int) -> L.IzhikevichParams:
    tau, v_th, v_reset, v_rest, v_c, a0, tau_w, a, b = scalars
    return L.IzhikevichParams(tau, v_th, v_reset, v_rest, v_c, a0, tau_w, a, b, sg_alpha, sg_id, flags)


def _flags(soft_reset: bool, detach_reset: bool, mode_flags: int) -> int:
    return ((int(mode_flags) & L.FLAG_FP32_STATE) | (L.FLAG_SOFT_RESET if soft_reset else 0)
            | (L.FLAG_DETACH_RESET if detach_reset else 0))


@torch.library.custom_op("sj::hip_multistep_izhikevich_forward", mutates_args=())
def hip_multistep_izhikevich_forward(x_seq: torch.Tensor, v_init: torch.Tensor, w_init: torch.Tensor,
                                     scalars: list[float], soft_reset: bool, detach_reset: bool, sg_id: int,
                                     sg_alpha: float, store_v_seq: bool, store_w_seq: bool, save_h: bool,
                                     mode_flags: int, replay: bool = False
                                     ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                                                torch.Tensor]:
    """``scalars`` = [tau, v_threshold, v_reset, v_rest, v_c, a0, tau_w, a, b].  ``replay``: a gradient, if one is
    asked for, is computed by the replaying backward, so ``save_h`` is not needed for it."""
    for name, t in (("x_seq", x_seq), ("v_init", v_init), ("w_init", w_init)):
        L.require_device_tensor(name, t)
    if x_seq.dim() != 2 or x_seq.shape[0] < 1 or x_seq.shape[1] < 1:
        raise ValueError(f"x_seq must be [T, N] with T, N >= 1, got shape {tuple(x_seq.shape)}")
    for name, t in (("v_init", v_init), ("w_init", w_init)):
        if t.shape != x_seq.shape[1:] or t.dtype != x_seq.dtype:
            raise ValueError(f"{name} must have shape {tuple(x_seq.shape[1:])} and dtype {x_seq.dtype}")
    dtype = L.dtype_id(x_seq.dtype)
    x_seq = x_seq.contiguous()
    T, N = x_seq.shape
    v_init, v_flag = _state_arg(v_init, False)
    w_init, w_flag = _state_arg(w_init, False)
    flags = _flags(soft_reset, detach_reset, mode_flags) | v_flag | (L.FLAG_W_INIT_BROADCAST if w_flag else 0)
    spike_seq = torch.empty_like(x_seq)
    # outputs of an operator may not alias each other: every unused one is its own empty tensor
    v_seq = torch.empty_like(x_seq) if store_v_seq else x_seq.new_empty((0,))
    w_seq = torch.empty_like(x_seq) if store_w_seq else x_seq.new_empty((0,))
    h_seq = torch.empty_like(x_seq) if save_h else x_seq.new_empty((0,))
    v_last, w_last = x_seq.new_empty((N,)), x_seq.new_empty((N,))
    params = _params(scalars, 0, 0.0, flags)
    with torch.cuda.device(x_seq.device):
        rc = L.load().sjhip_izhikevich_forward(
            dtype, ctypes.byref(params), T, N, x_seq.data_ptr(), v_init.data_ptr(), w_init.data_ptr(),
            spike_seq.data_ptr(), v_seq.data_ptr() if store_v_seq else None,
            w_seq.data_ptr() if store_w_seq else None, v_last.data_ptr(), w_last.data_ptr(),
            h_seq.data_ptr() if save_h else None, L.current_stream_ptr(x_seq.device))
    L.check(rc, "izhikevich_forward")
    return spike_seq, v_seq, w_seq, v_last, w_last, h_seq


@hip_multistep_izhikevich_forward.register_fake
def _(x_seq, v_init, w_init, scalars, soft_reset, detach_reset, sg_id, sg_alpha, store_v_seq, store_w_seq, save_h,
      mode_flags, replay=False):
    return (x_seq.new_empty(x_seq.shape),
            x_seq.new_empty(x_seq.shape) if store_v_seq else x_seq.new_empty((0,)),
            x_seq.new_empty(x_seq.shape) if store_w_seq else x_seq.new_empty((0,)),
            v_init.new_empty(v_init.shape), v_init.new_empty(v_init.shape),
            x_seq.new_empty(x_seq.shape) if save_h else x_seq.new_empty((0,)))


@torch.library.custom_op("sj::hip_multistep_izhikevich_backward", mutates_args=())
def hip_multistep_izhikevich_backward(grad_spike_seq: Optional[torch.Tensor], grad_v_seq: Optional[torch.Tensor],
                                      grad_w_seq: Optional[torch.Tensor], grad_v_last: Optional[torch.Tensor],
                                      grad_w_last: Optional[torch.Tensor], h_seq: torch.Tensor, v_init: torch.Tensor,
                                      scalars: list[float], soft_reset: bool, detach_reset: bool, sg_id: int,
                                      sg_alpha: float, mode_flags: int
                                      ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    L.require_device_tensor("h_seq", h_seq)
    h_seq = h_seq.contiguous()
    dtype = L.dtype_id(h_seq.dtype)
    T, N = h_seq.shape
    fix = lambda t: None if t is None else t.to(h_seq.dtype).contiguous()
    grad_spike_seq = torch.zeros_like(h_seq) if grad_spike_seq is None else fix(grad_spike_seq)
    grad_v_seq, grad_w_seq, grad_v_last, grad_w_last = map(fix, (grad_v_seq, grad_w_seq, grad_v_last, grad_w_last))
    v_init, v_flag = _state_arg(v_init, False)
    params = _params(scalars, sg_id, sg_alpha, _flags(soft_reset, detach_reset, mode_flags) | v_flag)
    grad_x = torch.empty_like(h_seq)
    grad_v_init, grad_w_init = h_seq.new_empty((N,)), h_seq.new_empty((N,))
    with torch.cuda.device(h_seq.device):
        rc = L.load().sjhip_izhikevich_backward(
            dtype, ctypes.byref(params), T, N, grad_spike_seq.data_ptr(), L.ptr(grad_v_seq), L.ptr(grad_w_seq),
            L.ptr(grad_v_last), L.ptr(grad_w_last), h_seq.data_ptr(), v_init.data_ptr(),
            grad_x.data_ptr(), grad_v_init.data_ptr(), grad_w_init.data_ptr(), L.current_stream_ptr(h_seq.device))
    L.check(rc, "izhikevich_backward")
    return grad_x, grad_v_init, grad_w_init


@hip_multistep_izhikevich_backward.register_fake
def _(grad_spike_seq, grad_v_seq, grad_w_seq, grad_v_last, grad_w_last, h_seq, v_init, scalars, soft_reset, detach_reset,
      sg_id, sg_alpha, mode_flags):
    return torch.empty_like(h_seq), h_seq.new_empty(h_seq.shape[1:]), h_seq.new_empty(h_seq.shape[1:])


@torch.library.custom_op("sj::hip_multistep_izhikevich_backward_replay", mutates_args=())
def hip_multistep_izhikevich_backward_replay(grad_spike_seq: Optional[torch.Tensor], grad_v_seq: Optional[torch.Tensor],
                                             grad_w_seq: Optional[torch.Tensor], grad_v_last: Optional[torch.Tensor],
                                             grad_w_last: Optional[torch.Tensor], x_seq: torch.Tensor,
                                             v_init: torch.Tensor, w_init: torch.Tensor, scalars: list[float],
                                             soft_reset: bool, detach_reset: bool, sg_id: int, sg_alpha: float,
                                             mode_flags: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    L.require_device_tensor("x_seq", x_seq)
    x_seq = L.aligned16(x_seq)  # the replay kernel has only the 128-bit path
    dtype = L.dtype_id(x_seq.dtype)
    T, N = x_seq.shape
    fix = lambda t: None if t is None else L.aligned16(t.to(x_seq.dtype))
    grad_spike_seq = torch.zeros_like(x_seq) if grad_spike_seq is None else fix(grad_spike_seq)
    grad_v_seq, grad_w_seq, grad_v_last, grad_w_last = map(fix, (grad_v_seq, grad_w_seq, grad_v_last, grad_w_last))
    v_init, v_flag = _state_arg(v_init, True)
    w_init, w_flag = _state_arg(w_init, True)
    flags = _flags(soft_reset, detach_reset, mode_flags) | v_flag | (L.FLAG_W_INIT_BROADCAST if w_flag else 0)
    params = _params(scalars, sg_id, sg_alpha, flags)
    grad_x = torch.empty_like(x_seq)
    grad_v_init, grad_w_init = x_seq.new_empty((N,)), x_seq.new_empty((N,))
    with torch.cuda.device(x_seq.device):
        rc = L.load().sjhip_izhikevich_backward_replay(
            dtype, ctypes.byref(params), T, N, x_seq.data_ptr(), v_init.data_ptr(), w_init.data_ptr(),
            grad_spike_seq.data_ptr(), L.ptr(grad_v_seq), L.ptr(grad_w_seq), L.ptr(grad_v_last), L.ptr(grad_w_last),
            grad_x.data_ptr(), grad_v_init.data_ptr(), grad_w_init.data_ptr(), L.current_stream_ptr(x_seq.device))
    L.check(rc, "izhikevich_backward(replay)")
    return grad_x, grad_v_init, grad_w_init


@hip_multistep_izhikevich_backward_replay.register_fake
def _(grad_spike_seq, grad_v_seq, grad_w_seq, grad_v_last, grad_w_last, x_seq, v_init, w_init, scalars, soft_reset,
      detach_reset, sg_id, sg_alpha, mode_flags):
    return torch.empty_like(x_seq), x_seq.new_empty(x_seq.shape[1:]), x_seq.new_empty(x_seq.shape[1:])


def _setup_context(ctx, inputs, output):
    (x_seq, v_init, w_init, scalars, soft_reset, detach_reset, sg_id, sg_alpha, store_v_seq, store_w_seq, save_h,
     mode_flags, replay) = inputs
    if replay:
        ctx.save_for_backward(x_seq, v_init, w_init)
    elif save_h:
        ctx.save_for_backward(output[5], v_init)
    else:
        raise RuntimeError("hip_multistep_izhikevich_forward was called with neither save_h nor replay but needs a "
                           "gradient")
    ctx.replay = replay
    ctx.scalars = (list(scalars), soft_reset, detach_reset, sg_id, sg_alpha, mode_flags)
    ctx.store_seq = (store_v_seq, store_w_seq)
    ctx.set_materialize_grads(False)


def _backward(ctx, grad_spike_seq, grad_v_seq, grad_w_seq, grad_v_last, grad_w_last, grad_h_seq):
    del grad_h_seq
    if not ctx.store_seq[0]:
        grad_v_seq = None
    if not ctx.store_seq[1]:
        grad_w_seq = None
    if ctx.replay:
        x_seq, v_init, w_init = ctx.saved_tensors
        gx, gv, gw = hip_multistep_izhikevich_backward_replay(grad_spike_seq, grad_v_seq, grad_w_seq, grad_v_last,
                                                              grad_w_last, x_seq, v_init, w_init, *ctx.scalars)
    else:
        h_seq, v_init = ctx.saved_tensors
        gx, gv, gw = hip_multistep_izhikevich_backward(grad_spike_seq, grad_v_seq, grad_w_seq, grad_v_last, grad_w_last,
                                                       h_seq, v_init, *ctx.scalars)
    return (gx, gv if ctx.needs_input_grad[1] else None, gw if ctx.needs_input_grad[2] else None) + (None,) * 10


torch.library.register_autograd("sj::hip_multistep_izhikevich_forward", _backward, setup_context=_setup_context)
