"""Leaky integrate-and-fire neuron (reference ``neuron/lif.py:97-398``)."""

from __future__ import annotations

from typing import Optional

from .. import functional, surrogate
from .base_node import BaseNode


class LIFNode(BaseNode):
    """``h = v + (x - (v - v_reset))/tau`` (``decay_input=True``) or ``h = v - (v - v_reset)/tau + x``.

    Both step modes support ``backend='torch'`` and ``backend='hip'``.
    """

    def __init__(self, tau: float = 2.0, decay_input: bool = True, v_threshold: float = 1.0,
                 v_reset: Optional[float] = 0.0,
                 surrogate_function: surrogate.SurrogateFunctionBase = surrogate.Sigmoid(),
                 detach_reset: bool = False, step_mode="s", backend="torch", store_v_seq: bool = False):
        assert isinstance(tau, float) and tau > 1.0
        super().__init__(v_threshold, v_reset, surrogate_function, detach_reset, step_mode, backend, store_v_seq)
        self.tau = tau
        self.decay_input = decay_input

    @property
    def supported_backends(self):
        if self.step_mode in ("s", "m"):
            return ("torch", "hip")
        raise ValueError(self.step_mode)

    def extra_repr(self):
        return super().extra_repr() + f", tau={self.tau}"

    def single_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend == "hip":
            self._check_hip_surrogate()
            spike, v = functional.lif_step_hip(inputs[0], states[0], self.tau, self.decay_input, self.v_threshold,
                                               self.v_reset, self.surrogate_function, self.detach_reset)
        elif self.backend == "torch":
            spike, v = functional.lif_step(inputs[0], states[0], self.tau, self.decay_input, self.v_threshold,
                                           self.v_reset, self._torch_surrogate(), self.detach_reset)
        else:
            raise ValueError(self.backend)
        return (spike,), (v, *states[1:])

    def _hip_multi_step(self, x_seq, v, store_v_seq):
        return functional.lif_multi_step_hip(x_seq, v, self.tau, self.decay_input, self.v_threshold,
                                             self.v_reset, self.surrogate_function, self.detach_reset,
                                             store_v_seq)
