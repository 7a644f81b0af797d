"""Surrogate gradient functions.

Forward of a *spiking* surrogate is the Heaviside step; its backward is the derivative of a
smooth primitive.  Counterpart of the reference's ``spikingjelly/activation_based/surrogate.py``
for the surrogates the kernel backends know (ids as in
``triton_kernel/surrogate_kernel.py:26-34``): ``Sigmoid`` (:769-933), ``ATan`` (:1247-1412),
``PiecewiseQuadratic`` (:401-592), ``PiecewiseExp`` (:595-766), ``SoftSign`` (:936-1098),
``SuperSpike`` (:1101-1244), ``Erf`` (:1610-1783), plus ``PiecewiseLeakyReLU`` (:1786-2001) as
a torch-only surrogate the hip backend must reject by name, and ``MultiLevelSpikeCount`` (:3107-3160),
the integer firing function of ``ILIFNode``.
"""

from __future__ import annotations

import math
import numbers

import torch
import torch.nn as nn
import torch.nn.functional as F

__all__ = [
    "heaviside",
    "SurrogateFunctionBase",
    "Sigmoid",
    "ATan",
    "PiecewiseQuadratic",
    "PiecewiseExp",
    "SoftSign",
    "SuperSpike",
    "Erf",
    "PiecewiseLeakyReLU",
    "MultiLevelSpikeCount",
]


def heaviside(x: torch.Tensor) -> torch.Tensor:
    """``1`` where ``x >= 0`` else ``0``, in ``x``'s dtype (reference surrogate.py:12-60)."""
    return (x >= 0).to(x)


class SurrogateFunctionBase(nn.Module):
    """Callable surrogate: ``spiking=True`` -> Heaviside forward with surrogate backward,
    ``spiking=False`` -> the smooth primitive itself.  Keyword parameters (``alpha`` ...)
    become attributes and are listed in ``_sg_param_names`` (reference surrogate.py:291-398)."""

    def __init__(self, spiking=True, **kwargs):
        super().__init__()
        self.spiking = spiking
        self._sg_param_names = tuple(kwargs.keys())
        for name, value in kwargs.items():
            setattr(self, name, value)

    def set_spiking_mode(self, spiking: bool):
        self.spiking = spiking

    @property
    def _sg_params(self) -> dict:
        return {name: getattr(self, name) for name in self._sg_param_names}

    def extra_repr(self):
        parts = [f"{k}={v}" for k, v in self._sg_params.items()]
        parts.append(f"spiking={self.spiking}")
        return ", ".join(parts)

    @staticmethod
    def spiking_function(x, **kwargs):
        raise NotImplementedError

    @staticmethod
    def primitive_function(x, **kwargs):
        raise NotImplementedError

    def forward(self, x: torch.Tensor):
        if self.spiking:
            return self.spiking_function(x, **self._sg_params)
        return self.primitive_function(x, **self._sg_params)


def _make_spiking_function(name: str, backward_fn):
    """autograd.Function: Heaviside forward, ``backward_fn(grad, x, *params)`` backward."""

    class _Fn(torch.autograd.Function):
        @staticmethod
        def forward(x, *params):
            return heaviside(x)

        @staticmethod
        def setup_context(ctx, inputs, output):
            ctx.save_for_backward(inputs[0])
            ctx.params = inputs[1:]

        @staticmethod
        def backward(ctx, grad_output):
            (x,) = ctx.saved_tensors
            return (backward_fn(grad_output, x, *ctx.params),) + (None,) * len(ctx.params)

    _Fn.__name__ = _Fn.__qualname__ = name
    return _Fn


# ---- Sigmoid -----------------------------------------------------------------------------------
def sigmoid_backward(grad_output: torch.Tensor, x: torch.Tensor, alpha: float):
    s = (x * alpha).sigmoid_()
    return grad_output * (1.0 - s) * s * alpha


sigmoid = _make_spiking_function("sigmoid", sigmoid_backward)


class Sigmoid(SurrogateFunctionBase):
    """g(x) = sigmoid(alpha x);  g'(x) = alpha g (1 - g)."""

    def __init__(self, alpha=4.0, spiking=True):
        super().__init__(spiking=spiking, alpha=alpha)

    @staticmethod
    def spiking_function(x, alpha):
        return sigmoid.apply(x, alpha)

    @staticmethod
    def primitive_function(x, alpha):
        return (x * alpha).sigmoid()

    @staticmethod
    def backward(grad_output, x, alpha):
        return sigmoid_backward(grad_output, x, alpha)


# ---- ATan --------------------------------------------------------------------------------------
def atan_backward(grad_output: torch.Tensor, x: torch.Tensor, alpha: float):
    a = alpha / 2
    ax = math.pi * a * x
    return a / (1 + ax * ax) * grad_output


atan = _make_spiking_function("atan", atan_backward)


class ATan(SurrogateFunctionBase):
    """g(x) = atan(pi/2 alpha x)/pi + 1/2;  g'(x) = (alpha/2) / (1 + (pi/2 alpha x)^2)."""

    def __init__(self, alpha=2.0, spiking=True):
        super().__init__(spiking=spiking, alpha=alpha)

    @staticmethod
    def spiking_function(x, alpha):
        return atan.apply(x, alpha)

    @staticmethod
    def primitive_function(x, alpha):
        return (math.pi / 2 * alpha * x).atan_() / math.pi + 0.5

    @staticmethod
    def backward(grad_output, x, alpha):
        return atan_backward(grad_output, x, alpha)


# ---- PiecewiseQuadratic ------------------------------------------------------------------------
def piecewise_quadratic_backward(grad_output: torch.Tensor, x: torch.Tensor, alpha: float):
    x_abs = x.abs()
    outside = x_abs > (1 / alpha)
    return (grad_output * (-(alpha**2) * x_abs + alpha)).masked_fill_(outside, 0)


piecewise_quadratic = _make_spiking_function("piecewise_quadratic", piecewise_quadratic_backward)


class PiecewiseQuadratic(SurrogateFunctionBase):
    """g'(x) = max(0, alpha - alpha^2 |x|)."""

    def __init__(self, alpha=1.0, spiking=True):
        super().__init__(spiking=spiking, alpha=alpha)

    @staticmethod
    def spiking_function(x, alpha):
        return piecewise_quadratic.apply(x, alpha)

    @staticmethod
    def primitive_function(x, alpha):
        above = (x > (1.0 / alpha)).to(x)
        inside = (x.abs() <= (1.0 / alpha)).to(x)
        return above + inside * (-(alpha**2) / 2 * x.square() * x.sign() + alpha * x + 0.5)

    @staticmethod
    def backward(grad_output, x, alpha):
        return piecewise_quadratic_backward(grad_output, x, alpha)


# ---- PiecewiseExp ------------------------------------------------------------------------------
def piecewise_exp_backward(grad_output: torch.Tensor, x: torch.Tensor, alpha: float):
    return alpha / 2 * (-alpha * x.abs()).exp_() * grad_output


piecewise_exp = _make_spiking_function("piecewise_exp", piecewise_exp_backward)


class PiecewiseExp(SurrogateFunctionBase):
    """g'(x) = alpha/2 exp(-alpha |x|)."""

    def __init__(self, alpha=1.0, spiking=True):
        super().__init__(spiking=spiking, alpha=alpha)

    @staticmethod
    def spiking_function(x, alpha):
        return piecewise_exp.apply(x, alpha)

    @staticmethod
    def primitive_function(x, alpha):
        nonneg = heaviside(x)
        sign = nonneg * 2.0 - 1.0
        tail = (sign * x * -alpha).exp_() / 2.0
        return nonneg - tail * sign

    @staticmethod
    def backward(grad_output, x, alpha):
        return piecewise_exp_backward(grad_output, x, alpha)


# ---- SoftSign ----------------------------------------------------------------------------------
def soft_sign_backward(grad_output: torch.Tensor, x: torch.Tensor, alpha: float):
    return grad_output / (2 * alpha * (1 / alpha + x.abs()).pow_(2))


soft_sign = _make_spiking_function("soft_sign", soft_sign_backward)


class SoftSign(SurrogateFunctionBase):
    """g(x) = (softsign(alpha x) + 1)/2;  g'(x) = 1 / (2 alpha (1/alpha + |x|)^2)."""

    def __init__(self, alpha=2.0, spiking=True):
        super().__init__(spiking=spiking, alpha=alpha)
        assert alpha > 0, "alpha must be lager than 0"

    @staticmethod
    def spiking_function(x, alpha):
        return soft_sign.apply(x, alpha)

    @staticmethod
    def primitive_function(x, alpha):
        return (F.softsign(x * alpha) + 1.0) / 2.0

    @staticmethod
    def backward(grad_output, x, alpha):
        return soft_sign_backward(grad_output, x, alpha)


# ---- SuperSpike --------------------------------------------------------------------------------
def super_spike_backward(grad_output: torch.Tensor, x: torch.Tensor, alpha: float):
    return alpha * grad_output / torch.pow(torch.abs(x) + 1.0, 2)


super_spike = _make_spiking_function("super_spike", super_spike_backward)


class SuperSpike(SurrogateFunctionBase):
    """g'(x) = alpha / (|x| + 1)^2; there is no primitive (reference surrogate.py:1236-1237)."""

    def __init__(self, alpha=1.0, spiking=True):
        super().__init__(spiking=spiking, alpha=alpha)

    @staticmethod
    def spiking_function(x, alpha):
        return super_spike.apply(x, alpha)

    @staticmethod
    def primitive_function(x, alpha):
        raise NotImplementedError

    @staticmethod
    def backward(grad_output, x, alpha):
        return super_spike_backward(grad_output, x, alpha)


# ---- Erf ---------------------------------------------------------------------------------------
def erf_backward(grad_output: torch.Tensor, x: torch.Tensor, alpha: float):
    return grad_output * (-(x * alpha).pow_(2)).exp_() * (alpha / math.sqrt(math.pi))


erf = _make_spiking_function("erf", erf_backward)


class Erf(SurrogateFunctionBase):
    """g(x) = erfc(-alpha x)/2;  g'(x) = alpha/sqrt(pi) exp(-(alpha x)^2)."""

    def __init__(self, alpha=2.0, spiking=True):
        super().__init__(spiking=spiking, alpha=alpha)

    @staticmethod
    def spiking_function(x, alpha):
        return erf.apply(x, alpha)

    @staticmethod
    def primitive_function(x, alpha):
        return torch.erfc_(-alpha * x) / 2.0

    @staticmethod
    def backward(grad_output, x, alpha):
        return erf_backward(grad_output, x, alpha)


# ---- PiecewiseLeakyReLU (torch backend only) ---------------------------------------------------
def piecewise_leaky_relu_backward(grad_output: torch.Tensor, x: torch.Tensor, w: float, c: float):
    inside = x.abs() < w
    slope = x.masked_fill(inside, 1 / (2 * w)).masked_fill(inside.logical_not(), c)
    return grad_output * slope


piecewise_leaky_relu = _make_spiking_function("piecewise_leaky_relu", piecewise_leaky_relu_backward)


class PiecewiseLeakyReLU(SurrogateFunctionBase):
    """g'(x) = 1/(2w) for |x| < w else c.  Not available in the kernel backends."""

    def __init__(self, w=1.0, c=0.01, spiking=True):
        super().__init__(spiking=spiking, w=w, c=c)

    @staticmethod
    def spiking_function(x, w, c):
        return piecewise_leaky_relu.apply(x, w, c)

    @staticmethod
    def primitive_function(x, w, c):
        below = (x < -w).to(x)
        above = (x > w).to(x)
        middle = torch.ones_like(x.data) - below - above
        if c == 0:
            return middle * (x / (2 * w) + 1 / 2) + above
        cw = c * w
        return below * (c * x + cw) + above * (c * x + (-cw + 1)) + middle * (x / (2 * w) + 1 / 2)

    @staticmethod
    def backward(grad_output, x, w, c):
        return piecewise_leaky_relu_backward(grad_output, x, w, c)


# ---- multi-level spike count (ILIF) ---------------------------------------------------------------
class MultiLevelSpikeCount(SurrogateFunctionBase):
    """Firing function of the integer-valued LIF: spiking -> ``round(clamp(x, 0, max_spike_count))`` with a
    rectangular straight-through gradient on ``grad_window`` (default ``[0, max_spike_count]``); not spiking ->
    ``clamp(x, 0, max_spike_count)``.  ``x`` is the charged voltage divided by the threshold."""

    def __init__(self, max_spike_count: int, grad_window=None, spiking: bool = True):
        if isinstance(max_spike_count, bool) or not isinstance(max_spike_count, numbers.Integral):
            raise TypeError("max_spike_count must be an integer.")
        max_spike_count = int(max_spike_count)
        if max_spike_count < 1:
            raise ValueError("max_spike_count must be >= 1.")
        if grad_window is None:
            grad_min, grad_max = 0.0, float(max_spike_count)
        else:
            grad_min, grad_max = grad_window
            if grad_min > grad_max:
                raise ValueError("grad_window must satisfy grad_min <= grad_max.")
        super().__init__(spiking=spiking, max_spike_count=max_spike_count, grad_min=grad_min, grad_max=grad_max)

    @staticmethod
    def spiking_function(x: torch.Tensor, max_spike_count: int, grad_min: float, grad_max: float):
        from . import quantize

        return quantize.multi_level_spike_count(x, max_spike_count, (grad_min, grad_max))

    @staticmethod
    def primitive_function(x: torch.Tensor, max_spike_count: int, grad_min: float, grad_max: float):
        del grad_min, grad_max
        return torch.clamp(x, 0, max_spike_count)
