"""Activation-aware IF neuron (reference ``neuron/integrate_and_fire.py:536-1150``)."""

from __future__ import annotations

from typing import Optional, Union

import torch

from .. import base, functional, surrogate

__all__ = ["ActivationAwareIFNode"]


class ActivationAwareIFNode(base.MemoryModule):
    """IF neuron of the activation-aware redistribution style of ANN2SNN conversion: it fires on
    ``h + v_offset >= v_threshold`` with ``v_threshold`` (finite, positive) and ``v_offset`` (finite) either scalars or
    1-D tensors over the axis ``channel_dim`` of one time step.  Soft reset subtracts the channel's threshold, hard
    reset goes to ``v_reset``.

    ``backend='torch'`` serves both step modes and training.  ``backend='hip'`` serves multi-step inference only, as
    the reference's ``'triton'`` backend does: it refuses training mode, gradients, non-spiking surrogates and CPU
    tensors instead of falling back.
    """

    def __init__(self, v_threshold: Union[float, torch.Tensor] = 1.0, v_offset: Union[float, torch.Tensor] = 0.0,
                 channel_dim: int = -1, v_reset: Optional[float] = None,
                 surrogate_function: surrogate.SurrogateFunctionBase = surrogate.Sigmoid(),
                 detach_reset: bool = False, step_mode: str = "s", backend: str = "torch", store_v_seq: bool = False):
        super().__init__()
        if backend not in ("torch", "hip"):
            raise ValueError(f"Unsupported backend={backend!r}.")
        if backend == "hip" and step_mode != "m":
            raise ValueError("ActivationAwareIFNode backend='hip' requires step_mode='m'.")
        if v_reset is not None and not isinstance(v_reset, float):
            raise ValueError(f"v_reset must be a float or None, got {type(v_reset).__name__}.")
        if not isinstance(detach_reset, bool):
            raise ValueError("detach_reset must be bool.")
        if not isinstance(store_v_seq, bool):
            raise ValueError("store_v_seq must be bool.")
        if not isinstance(channel_dim, int):
            raise ValueError("channel_dim must be int.")
        threshold, offset = torch.as_tensor(v_threshold), torch.as_tensor(v_offset)
        self._check_parameter("v_threshold", threshold, positive=True)
        self._check_parameter("v_offset", offset, positive=False)
        self.register_buffer("v_threshold", threshold.clone().detach())
        self.register_buffer("v_offset", offset.clone().detach())
        self.channel_dim = channel_dim
        self.v_reset = v_reset
        self.detach_reset = detach_reset
        self.surrogate_function = surrogate_function
        self.register_memory("v", 0.0 if v_reset is None else v_reset)
        self.store_v_seq = store_v_seq
        self.step_mode = step_mode
        self.backend = backend

    @staticmethod
    def _check_parameter(name: str, value: torch.Tensor, positive: bool) -> None:
        if value.dim() > 1:
            raise ValueError(f"{name} must be a scalar or 1D tensor, but got shape {tuple(value.shape)}.")
        value = value if torch.is_floating_point(value) else value.to(torch.float)
        if not torch.isfinite(value).all() or (positive and not (value > 0).all()):
            raise ValueError(f"{name} must contain finite{' positive' if positive else ''} values.")

    @property
    def supported_backends(self):
        return ("torch",) if self.step_mode == "s" else ("torch", "hip")

    @property
    def store_v_seq(self) -> bool:
        return self._store_v_seq

    @store_v_seq.setter
    def store_v_seq(self, value: bool) -> None:
        self._store_v_seq = value
        self.v_seq = None

    def reset(self):
        super().reset()
        self.v_seq = None

    def extra_repr(self):
        return (f"v_threshold_shape={tuple(self.v_threshold.shape)}, v_offset_shape={tuple(self.v_offset.shape)}, "
                f"channel_dim={self.channel_dim}, v_reset={self.v_reset}, detach_reset={self.detach_reset}, "
                f"step_mode={self.step_mode}, backend={self.backend}")

    # ---- channel handling -------------------------------------------------------------------------------
    def _canonical_channel_dim(self, x: torch.Tensor) -> int:
        dim = self.channel_dim + x.dim() if self.channel_dim < 0 else self.channel_dim
        if dim < 0 or dim >= x.dim():
            raise ValueError(f"channel_dim={self.channel_dim} is out of range for input with {x.dim()} dimensions.")
        return dim

    def _check_length(self, name: str, param: torch.Tensor, x: torch.Tensor) -> None:
        channels = x.shape[self._canonical_channel_dim(x)]
        if param.numel() != channels:
            raise ValueError(f"{name} has length {param.numel()}, but input shape {tuple(x.shape)} has {channels} "
                             f"channels at channel_dim={self.channel_dim}.")

    def _broadcast_parameter(self, param: torch.Tensor, x: torch.Tensor, name: str) -> torch.Tensor:
        param = param.to(device=x.device, dtype=x.dtype)
        if param.dim() == 0:
            return param
        self._check_length(name, param, x)
        shape = [1] * x.dim()
        shape[self._canonical_channel_dim(x)] = param.numel()
        return param.view(shape)

    # ---- forward ----------------------------------------------------------------------------------------
    def materialize_states(self, inputs, states, step_mode: str):
        x = inputs[0][0] if step_mode == "m" else inputs[0]
        v = states[0]
        start = self.v_reset if self.v_reset is not None else 0.0
        if isinstance(v, float):
            v = self._fresh(x, v)
        elif isinstance(v, torch.Tensor):
            if v.shape != x.shape:
                v = self._fresh(x, start)
            elif v.dtype != x.dtype or v.device != x.device:
                v = v.to(dtype=x.dtype, device=x.device)
        return (v, *states[1:])

    def _fresh(self, x: torch.Tensor, value: float) -> torch.Tensor:
        # the hip kernel reads a constant state from one element: no [N] tensor is filled or read
        if self.backend == "hip" and x.is_cuda and x.numel() > 1:
            return x.new_full((1,) * x.dim(), value).expand(x.shape)
        return torch.full_like(x, value, requires_grad=False)

    def single_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend != "torch":
            raise RuntimeError("ActivationAwareIFNode single-step forward supports only backend='torch'; "
                               "refusing implicit backend fallback.")
        x, v = inputs[0], states[0]
        spike, v = functional.activation_aware_if_step(
            x, v, self._broadcast_parameter(self.v_threshold, x, "v_threshold"),
            self._broadcast_parameter(self.v_offset, x, "v_offset"), self.v_reset, self.surrogate_function,
            self.detach_reset)
        return (spike,), (v, *states[1:])

    def _hip_multi_step(self, x_seq: torch.Tensor, v, store_v_seq: bool):
        if x_seq.device.type != "cuda":
            raise RuntimeError("ActivationAwareIFNode backend='hip' requires a ROCm device tensor.")
        if self.training:
            raise RuntimeError("ActivationAwareIFNode backend='hip' supports inference only; call eval() before forward.")
        if not getattr(self.surrogate_function, "spiking", True):
            raise RuntimeError("ActivationAwareIFNode backend='hip' requires a spiking surrogate function.")
        if torch.is_grad_enabled() and any(t.requires_grad for t in (x_seq, v, self.v_threshold, self.v_offset)
                                           if isinstance(t, torch.Tensor)):
            raise RuntimeError("ActivationAwareIFNode backend='hip' does not support autograd.")
        step = x_seq[0]
        if self.v_threshold.dim() == 1 or self.v_offset.dim() == 1:
            dim = self._canonical_channel_dim(step)
            for name, param in (("v_threshold", self.v_threshold), ("v_offset", self.v_offset)):
                if param.dim() == 1:
                    self._check_length(name, param, step)
            channel_size = step.shape[dim]
            inner_size = 1
            for size in step.shape[dim + 1:]:
                inner_size *= size
        else:
            channel_size, inner_size = 1, step.numel()
        return functional.activation_aware_if_multi_step_hip(x_seq, v, self.v_threshold, self.v_offset, channel_size,
                                                             inner_size, self.v_reset, store_v_seq)

    def multi_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend == "hip":
            spike_seq, v, _ = self._hip_multi_step(inputs[0], states[0], False)
            return (spike_seq,), (v,)
        if self.backend == "torch":
            return super().multi_step_functional_forward(inputs, states, **kwargs)
        raise ValueError(self.backend)

    def multi_step_forward(self, x_seq: torch.Tensor, *args, **kwargs):
        if not self.store_v_seq:
            return super().multi_step_forward(x_seq, *args, **kwargs)
        states = self.materialize_states((x_seq, *args), tuple(self._memories.values()), "m")
        if self.backend == "hip":
            spike_seq, v, v_seq = self._hip_multi_step(x_seq, states[0], True)
        elif self.backend == "torch":
            spikes, voltages = [], []
            for t in range(x_seq.shape[0]):
                outputs, states = self.single_step_functional_forward((x_seq[t],), states, **kwargs)
                spikes.append(outputs[0])
                voltages.append(states[0])
            spike_seq, v, v_seq = torch.stack(spikes), states[0], torch.stack(voltages)
        else:
            raise ValueError(self.backend)
        self.v = v
        self.v_seq = v_seq
        return spike_seq
