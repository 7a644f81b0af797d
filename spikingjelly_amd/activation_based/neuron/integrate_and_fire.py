"""Integrate-and-fire neuron (reference ``neuron/integrate_and_fire.py:120-369``)."""

from __future__ import annotations

from typing import Optional

from .. import functional, surrogate
from .base_node import BaseNode


class IFNode(BaseNode):
    """``h[t] = v[t-1] + x[t]``; fire where ``h >= v_threshold``; hard or soft reset.

    Both step modes support ``backend='torch'`` and ``backend='hip'``.
    """

    def __init__(self, v_threshold: float = 1.0, v_reset: Optional[float] = 0.0,
                 surrogate_function: surrogate.SurrogateFunctionBase = surrogate.Sigmoid(),
                 detach_reset: bool = False, step_mode="s", backend="torch", store_v_seq: bool = False):
        super().__init__(v_threshold, v_reset, surrogate_function, detach_reset, step_mode, backend, store_v_seq)

    @property
    def supported_backends(self):
        if self.step_mode in ("s", "m"):
            return ("torch", "hip")
        raise ValueError(self.step_mode)

    def single_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend == "hip":
            self._check_hip_surrogate()
            spike, v = functional.if_step_hip(inputs[0], states[0], self.v_threshold, self.v_reset,
                                              self.surrogate_function, self.detach_reset)
        elif self.backend == "torch":
            spike, v = functional.if_step(inputs[0], states[0], self.v_threshold, self.v_reset,
                                          self._torch_surrogate(), self.detach_reset)
        else:
            raise ValueError(self.backend)
        return (spike,), (v, *states[1:])

    def _hip_multi_step(self, x_seq, v, store_v_seq):
        return functional.if_multi_step_hip(x_seq, v, self.v_threshold, self.v_reset, self.surrogate_function,
                                            self.detach_reset, store_v_seq)
