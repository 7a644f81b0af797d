"""Neurons with an adaptation current: ``AdaptBaseNode`` and ``IzhikevichNode`` (reference ``neuron/adapt.py``)."""

from __future__ import annotations

from typing import Optional

import torch

from .. import functional, surrogate
from .base_node import BaseNode

__all__ = ["AdaptBaseNode", "IzhikevichNode"]


class AdaptBaseNode(BaseNode):
    """``BaseNode`` plus the adaptation current ``w`` as a second memory (starts at ``w_rest``; reference
    ``neuron/adapt.py:12-176``)."""

    def __init__(self, v_threshold: float = 1.0, v_reset: Optional[float] = 0.0, v_rest: float = 0.0, w_rest: float = 0.0,
                 tau_w: float = 2.0, a: float = 0.0, b: float = 0.0,
                 surrogate_function: surrogate.SurrogateFunctionBase = surrogate.Sigmoid(), detach_reset: bool = False,
                 step_mode="s", backend="torch", store_v_seq: bool = False):
        assert isinstance(w_rest, float) and isinstance(v_rest, float)
        assert isinstance(tau_w, float) and isinstance(a, float) and isinstance(b, float)
        super().__init__(v_threshold, v_reset, surrogate_function, detach_reset, step_mode, backend, store_v_seq)
        self.register_memory("w", w_rest)
        self.w_rest = w_rest
        self.v_rest = v_rest
        self.tau_w = tau_w
        self.a = a
        self.b = b

    def extra_repr(self):
        return (super().extra_repr() + f", v_rest={self.v_rest}, w_rest={self.w_rest}, tau_w={self.tau_w}, a={self.a}, "
                f"b={self.b}")

    def materialize_states(self, inputs, states, step_mode: str):
        states = super().materialize_states(inputs, states, step_mode)
        v, w = states[0], states[-1]
        if isinstance(w, float):
            w = self._constant_state(v, w)
        elif isinstance(w, torch.Tensor):
            if w.shape != v.shape:
                w = self._constant_state(v, self.w_rest)
            elif w.dtype != v.dtype or w.device != v.device:
                w = w.to(dtype=v.dtype, device=v.device)
        return (*states[:-1], w)


class IzhikevichNode(AdaptBaseNode):
    """``h = v + (x + a0 (v - v_rest)(v - v_c) - w) / tau``, ``w`` relaxing towards ``a (h - v_rest)`` with ``tau_w`` and
    jumping by ``b`` at a spike (reference ``neuron/adapt.py:178-399``).  Multi-step mode supports ``backend='torch'``
    and ``backend='hip'`` (the reference: ``'torch'`` and ``'cupy'``), single-step mode torch only."""

    def __init__(self, tau: float = 2.0, v_c: float = 0.8, a0: float = 1.0, v_threshold: float = 1.0,
                 v_reset: Optional[float] = 0.0, v_rest: float = -0.1, w_rest: float = 0.0, tau_w: float = 2.0,
                 a: float = 0.0, b: float = 0.0, surrogate_function: surrogate.SurrogateFunctionBase = surrogate.Sigmoid(),
                 detach_reset: bool = False, step_mode="s", backend="torch", store_v_seq: bool = False):
        assert isinstance(tau, float) and tau > 1.0
        assert a0 > 0
        super().__init__(v_threshold, v_reset, v_rest, w_rest, tau_w, a, b, surrogate_function, detach_reset, step_mode,
                         backend, store_v_seq)
        self.tau = tau
        self.v_c = v_c
        self.a0 = a0

    def extra_repr(self):
        return super().extra_repr() + f", tau={self.tau}, v_c={self.v_c}, a0={self.a0}"

    @property
    def supported_backends(self):
        if self.step_mode == "s":
            return ("torch",)
        if self.step_mode == "m":
            return ("torch", "hip")
        raise ValueError(self.step_mode)

    def single_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend != "torch":
            raise ValueError(self.backend)
        spike, v, w = functional.izhikevich_step(inputs[0], states[0], states[-1], self.tau, self.a0, self.v_rest,
                                                 self.v_c, self.tau_w, self.a, self.b, self.v_threshold, self.v_reset,
                                                 self.surrogate_function, self.detach_reset)
        return (spike,), (v, w)

    def _hip(self, x_seq, v, w, store_state_seq: bool):
        return functional.izhikevich_multi_step_hip(x_seq, v, w, self.tau, self.v_threshold, self.v_reset, self.v_rest,
                                                    self.a, self.b, self.tau_w, self.v_c, self.a0, self.detach_reset,
                                                    self.surrogate_function, store_state_seq, False)

    def multi_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend == "hip":
            spike_seq, v, w, _, _ = self._hip(inputs[0], states[0], states[-1], False)
            return (spike_seq,), (v, w)
        if self.backend == "torch":
            return super(BaseNode, self).multi_step_functional_forward(inputs, states, **kwargs)
        raise ValueError(self.backend)

    def multi_step_forward(self, x_seq: torch.Tensor, *args, **kwargs):
        if not self.store_v_seq or self.backend != "hip":
            return super().multi_step_forward(x_seq, *args, **kwargs)
        states = self.materialize_states((x_seq, *args), tuple(self._memories.values()), "m")
        spike_seq, self.v, self.w, self.v_seq, _ = self._hip(x_seq, states[0], states[-1], True)
        return spike_seq
