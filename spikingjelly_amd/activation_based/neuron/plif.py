"""Parametric LIF neuron with a learnable time constant (reference ``neuron/plif.py:14-261``)."""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn

from .. import functional, surrogate
from .base_node import BaseNode


class ParametricLIFNode(BaseNode):
    """LIF whose ``1/tau = sigmoid(w)`` is learned; ``w`` starts at ``-log(init_tau - 1)``.

    Both step modes support ``backend='torch'`` and ``backend='hip'``.  Unlike IF/LIF the torch
    backend keeps the surrogate in eval mode (reference neuron/plif.py:170-186).
    """

    def __init__(self, init_tau: float = 2.0, decay_input: bool = True, v_threshold: float = 1.0,
                 v_reset: Optional[float] = 0.0,
                 surrogate_function: surrogate.SurrogateFunctionBase = surrogate.Sigmoid(),
                 detach_reset: bool = False, step_mode="s", backend="torch", store_v_seq: bool = False):
        assert isinstance(init_tau, float) and init_tau > 1.0
        super().__init__(v_threshold, v_reset, surrogate_function, detach_reset, step_mode, backend, store_v_seq)
        self.decay_input = decay_input
        self.w = nn.Parameter(torch.as_tensor(-math.log(init_tau - 1.0)))

    @property
    def supported_backends(self):
        if self.step_mode in ("s", "m"):
            return ("torch", "hip")
        raise ValueError(self.step_mode)

    def extra_repr(self):
        with torch.no_grad():
            tau = 1.0 / self.w.sigmoid()
        return super().extra_repr() + f", tau={tau}"

    def single_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend == "hip":
            spike, v = functional.plif_step_hip(inputs[0], states[0], self.w, self.decay_input, self.v_threshold,
                                                self.v_reset, self.surrogate_function, self.detach_reset)
        elif self.backend == "torch":
            spike, v = functional.plif_step(inputs[0], states[0], self.w, self.decay_input, self.v_threshold,
                                            self.v_reset, self.surrogate_function, self.detach_reset)
        else:
            raise ValueError(self.backend)
        return (spike,), (v, *states[1:])

    def _check_hip_surrogate(self):
        # the reference PLIF dispatch has no eval-mode surrogate check (neuron/plif.py:188-236)
        return None

    def _hip_multi_step(self, x_seq, v, store_v_seq):
        return functional.plif_multi_step_hip(x_seq, v, self.w, self.decay_input, self.v_threshold,
                                              self.v_reset, self.surrogate_function, self.detach_reset,
                                              store_v_seq)
