"""Quadratic and exponential integrate-and-fire neurons (reference ``neuron/nonlinear_if.py:12-240, 243-473``)."""

from __future__ import annotations

from typing import Optional

from .. import functional, surrogate
from .base_node import BaseNode


class _NonlinearIFNode(BaseNode):
    """What QIF and EIF share: multi-step mode supports ``backend='torch'`` and ``backend='hip'`` (the reference:
    ``'torch'`` and ``'cupy'``), single-step mode is torch only as in the reference, and like the reference nodes
    the torch backend keeps the surrogate in eval mode."""

    @property
    def supported_backends(self):
        if self.step_mode == "s":
            return ("torch",)
        if self.step_mode == "m":
            return ("torch", "hip")
        raise ValueError(self.step_mode)

    def _torch_surrogate(self):
        return self.surrogate_function

    def _check_hip_surrogate(self):
        # the reference dispatch of these nodes has no eval-mode surrogate check (neuron/nonlinear_if.py:171-196)
        return None


class QIFNode(_NonlinearIFNode):
    """``h[t] = v[t-1] + (x[t] + a0 (v[t-1] - v_rest)(v[t-1] - v_c)) / tau``."""

    def __init__(self, tau: float = 2.0, v_c: float = 0.8, a0: float = 1.0, v_threshold: float = 1.0,
                 v_rest: float = 0.0, v_reset: Optional[float] = -0.1,
                 surrogate_function: surrogate.SurrogateFunctionBase = surrogate.Sigmoid(),
                 detach_reset: bool = False, step_mode="s", backend="torch", store_v_seq: bool = False):
        assert isinstance(tau, float) and tau > 1.0
        if v_reset is not None:
            assert v_threshold > v_reset
            assert v_rest >= v_reset
        assert a0 > 0
        super().__init__(v_threshold, v_reset, surrogate_function, detach_reset, step_mode, backend, store_v_seq)
        self.tau = tau
        self.v_c = v_c
        self.v_rest = v_rest
        self.a0 = a0

    def extra_repr(self):
        return super().extra_repr() + f", tau={self.tau}, v_c={self.v_c}, a0={self.a0}, v_rest={self.v_rest}"

    def single_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend != "torch":
            raise ValueError(self.backend)
        spike, v = functional.qif_step(inputs[0], states[0], self.tau, self.a0, self.v_rest, self.v_c,
                                       self.v_threshold, self.v_reset, self.surrogate_function, self.detach_reset)
        return (spike,), (v, *states[1:])

    def _hip_multi_step(self, x_seq, v, store_v_seq):
        return functional.qif_multi_step_hip(x_seq, v, self.tau, self.v_threshold, self.v_reset, self.v_rest,
                                             self.v_c, self.a0, self.detach_reset, self.surrogate_function,
                                             store_v_seq)


class EIFNode(_NonlinearIFNode):
    """``h[t] = v[t-1] + (x[t] + v_rest - v[t-1] + delta_T exp((v[t-1] - theta_rh) / delta_T)) / tau``.

    On the hip backend ``exp`` is the device library's: ``h`` agrees with the torch backend
    to rounding, and a spike can differ where ``h`` lands within that distance of the threshold.
    """

    def __init__(self, tau: float = 2.0, delta_T: float = 1.0, theta_rh: float = 0.8, v_threshold: float = 1.0,
                 v_rest: float = 0.0, v_reset: Optional[float] = -0.1,
                 surrogate_function: surrogate.SurrogateFunctionBase = surrogate.Sigmoid(),
                 detach_reset: bool = False, step_mode="s", backend="torch", store_v_seq: bool = False):
        assert isinstance(tau, float) and tau > 1.0
        if v_reset is not None:
            assert v_threshold > v_reset
            assert v_rest >= v_reset
        assert delta_T > 0
        super().__init__(v_threshold, v_reset, surrogate_function, detach_reset, step_mode, backend, store_v_seq)
        self.tau = tau
        self.v_rest = v_rest
        self.delta_T = delta_T
        self.theta_rh = theta_rh

    def extra_repr(self):
        return (super().extra_repr() + f", tau={self.tau}, delta_T={self.delta_T}, theta_rh={self.theta_rh}"
                f", v_rest={self.v_rest}")

    def single_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend != "torch":
            raise ValueError(self.backend)
        spike, v = functional.eif_step(inputs[0], states[0], self.tau, self.delta_T, self.theta_rh, self.v_rest,
                                       self.v_threshold, self.v_reset, self.surrogate_function, self.detach_reset)
        return (spike,), (v, *states[1:])

    def _hip_multi_step(self, x_seq, v, store_v_seq):
        return functional.eif_multi_step_hip(x_seq, v, self.tau, self.v_threshold, self.v_reset, self.v_rest,
                                             self.theta_rh, self.delta_T, self.detach_reset, self.surrogate_function,
                                             store_v_seq)
