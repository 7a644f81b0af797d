"""torch-ops restatement of the reference torch backend (CPU).  Test infrastructure only.

Every arithmetic line cites the reference line it follows (paths relative to
``spikingjelly/activation_based``).  Op order and scalar handling are kept exactly, because the
HIP kernels are compared bit for bit against what these ops produce on CPU tensors.
"""

from __future__ import annotations

import math
from typing import Callable, Optional

import torch

# ------------------------------------------------------------------------------------------------
# surrogate functions
# ------------------------------------------------------------------------------------------------


def heaviside(x: torch.Tensor) -> torch.Tensor:
    # surrogate.py:60
    return (x >= 0).to(x)


class _SigmoidSG(torch.autograd.Function):
    # surrogate.py:811-851 (forward = heaviside) with backward :769-771
    @staticmethod
    def forward(ctx, x, alpha):
        ctx.save_for_backward(x)
        ctx.alpha = alpha
        return heaviside(x)

    @staticmethod
    def backward(ctx, grad_output):
        (x,) = ctx.saved_tensors
        sgax = (x * ctx.alpha).sigmoid_()
        return grad_output * (1.0 - sgax) * sgax * ctx.alpha, None


class _ATanSG(torch.autograd.Function):
    # surrogate.py:1290-1330 with backward :1247-1250
    @staticmethod
    def forward(ctx, x, alpha):
        ctx.save_for_backward(x)
        ctx.alpha = alpha
        return heaviside(x)

    @staticmethod
    def backward(ctx, grad_output):
        (x,) = ctx.saved_tensors
        a = ctx.alpha / 2
        ax = math.pi * a * x
        return a / (1 + ax * ax) * grad_output, None


def _sg_backward_other(name: str, grad_output, x, alpha):
    if name == "piecewise_quadratic":  # surrogate.py:401-407
        x_abs = x.abs()
        mask = x_abs > (1 / alpha)
        return (grad_output * (-(alpha**2) * x_abs + alpha)).masked_fill_(mask, 0)
    if name == "piecewise_exp":  # surrogate.py:595-596
        return alpha / 2 * (-alpha * x.abs()).exp_() * grad_output
    if name == "soft_sign":  # surrogate.py:936-937
        return grad_output / (2 * alpha * (1 / alpha + x.abs()).pow_(2))
    if name == "super_spike":  # surrogate.py:1101-1102
        return alpha * grad_output / torch.pow(torch.abs(x) + 1.0, 2)
    if name == "erf":  # surrogate.py:1610-1613
        return grad_output * (-(x * alpha).pow_(2)).exp_() * (alpha / math.sqrt(math.pi))
    raise ValueError(name)


class _OtherSG(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, alpha, name):
        ctx.save_for_backward(x)
        ctx.alpha = alpha
        ctx.name = name
        return heaviside(x)

    @staticmethod
    def backward(ctx, grad_output):
        (x,) = ctx.saved_tensors
        return _sg_backward_other(ctx.name, grad_output, x, ctx.alpha), None, None


class _MultiLevelCount(torch.autograd.Function):
    # quantize.py:580-598: forward round(clamp(x, 0, D)), backward passes the gradient inside [grad_min, grad_max]
    @staticmethod
    def forward(ctx, x, max_spike_count, grad_min, grad_max):
        ctx.save_for_backward(x)
        ctx.grad_min = grad_min
        ctx.grad_max = grad_max
        return torch.round(torch.clamp(x, 0, max_spike_count))

    @staticmethod
    def backward(ctx, grad_output):
        (x,) = ctx.saved_tensors
        mask = (x >= ctx.grad_min) & (x <= ctx.grad_max)
        return grad_output * mask.to(grad_output.dtype), None, None, None


def multi_level_spike_count(max_spike_count: int, grad_window=None) -> Callable[[torch.Tensor], torch.Tensor]:
    """Firing function of ILIF (surrogate.py:3107-3160, quantize.py:601-616); default window [0, D]."""
    grad_min, grad_max = (0.0, float(max_spike_count)) if grad_window is None else grad_window
    return lambda x: _MultiLevelCount.apply(x, int(max_spike_count), grad_min, grad_max)


SG_NAMES = ("sigmoid", "atan", "piecewise_quadratic", "piecewise_exp", "soft_sign", "super_spike", "erf")
SG_IDS = {name: i for i, name in enumerate(SG_NAMES)}  # triton_kernel/surrogate_kernel.py:26-34
SG_DEFAULT_ALPHA = {"sigmoid": 4.0, "atan": 2.0, "piecewise_quadratic": 1.0, "piecewise_exp": 1.0,
                    "soft_sign": 2.0, "super_spike": 1.0, "erf": 2.0}


def surrogate(name: str, alpha: float, spiking: bool = True) -> Callable[[torch.Tensor], torch.Tensor]:
    """Callable like a reference surrogate module: spiking -> Heaviside forward + surrogate
    backward; not spiking -> the smooth primitive."""
    if spiking:
        if name == "sigmoid":
            return lambda x: _SigmoidSG.apply(x, alpha)
        if name == "atan":
            return lambda x: _ATanSG.apply(x, alpha)
        if name in SG_IDS:
            return lambda x: _OtherSG.apply(x, alpha, name)
        raise ValueError(name)
    return lambda x: primitive(name, x, alpha)


def primitive(name: str, x: torch.Tensor, alpha: float) -> torch.Tensor:
    if name == "sigmoid":  # surrogate.py:925-926
        return (x * alpha).sigmoid()
    if name == "atan":  # surrogate.py:1404-1405
        return (math.pi / 2 * alpha * x).atan_() / math.pi + 0.5
    if name == "piecewise_quadratic":  # surrogate.py:582-588
        mask0 = (x > (1.0 / alpha)).to(x)
        mask1 = (x.abs() <= (1.0 / alpha)).to(x)
        return mask0 + mask1 * (-(alpha**2) / 2 * x.square() * x.sign() + alpha * x + 0.5)
    if name == "piecewise_exp":  # surrogate.py:758-762
        mask_nonnegative = heaviside(x)
        mask_sign = mask_nonnegative * 2.0 - 1.0
        exp_x = (mask_sign * x * -alpha).exp_() / 2.0
        return mask_nonnegative - exp_x * mask_sign
    if name == "soft_sign":  # surrogate.py:1093-1094
        return (torch.nn.functional.softsign(x * alpha) + 1.0) / 2.0
    if name == "erf":  # surrogate.py:1778-1779
        return torch.erfc_(-alpha * x) / 2.0
    raise ValueError(f"{name} has no primitive")


def surrogate_grad(name: str, x: torch.Tensor, alpha: float) -> torch.Tensor:
    """g'(x) as the reference's backward computes it for grad_output = 1."""
    one = torch.ones_like(x)
    if name == "sigmoid":
        sgax = (x * alpha).sigmoid_()
        return one * (1.0 - sgax) * sgax * alpha
    if name == "atan":
        a = alpha / 2
        ax = math.pi * a * x
        return a / (1 + ax * ax) * one
    return _sg_backward_other(name, one, x, alpha)


# ------------------------------------------------------------------------------------------------
# one step
# ------------------------------------------------------------------------------------------------


def voltage_reset(v, spike, v_threshold: float, v_reset: Optional[float], detach_reset: bool):
    # functional/neuron.py:225-228
    spike_d = spike.detach() if detach_reset else spike
    if v_reset is None:
        return v - spike_d * v_threshold
    return spike_d * v_reset + (1.0 - spike_d) * v


def charge(kind: str, x, v, tau_or_w, decay_input: bool, v_reset: Optional[float]):
    if kind == "if":
        return v + x  # functional/neuron.py:310
    v_reset_value = 0.0 if v_reset is None else v_reset
    if kind == "lif":
        # functional/neuron.py:849-852
        if decay_input:
            return v + (x - (v - v_reset_value)) / tau_or_w
        return v - (v - v_reset_value) / tau_or_w + x
    if kind == "plif":
        # functional/neuron.py:1290-1295
        reciprocal_tau = tau_or_w.sigmoid()
        if decay_input:
            return v + (x - (v - v_reset_value)) * reciprocal_tau
        return v - (v - v_reset_value) * reciprocal_tau + x
    if kind == "plif_k":
        # same as "plif" but fed k = sigmoid(w) directly (what the kernel operators receive)
        if decay_input:
            return v + (x - (v - v_reset_value)) * tau_or_w
        return v - (v - v_reset_value) * tau_or_w + x
    if kind == "qif":
        # functional/neuron.py:397; tau_or_w = (tau, a0, v_rest, v_c)
        tau, a0, v_rest, v_c = tau_or_w
        return v + (x + a0 * (v - v_rest) * (v - v_c)) / tau
    if kind == "eif":
        # functional/neuron.py:483-485; tau_or_w = (tau, delta_t, theta_rh, v_rest)
        tau, delta_t, theta_rh, v_rest = tau_or_w
        return v + (x + v_rest - v + delta_t * torch.exp((v - theta_rh) / delta_t)) / tau
    raise ValueError(kind)


def step(kind: str, x, v, tau_or_w, decay_input: bool, v_threshold: float, v_reset: Optional[float],
         sg: Callable, detach_reset: bool):
    """(spike, v_next, h): functional/neuron.py:310-312, 931-933, 1296-1297; "ilif" :1097-1099 (sg is the
    multi-level count, fed h / v_threshold; decay_input and v_reset are fixed to False and None)."""
    if kind == "ilif":
        h = charge("lif", x, v, tau_or_w, False, None)
        spike = sg(h / v_threshold)
        return spike, voltage_reset(h, spike, v_threshold, None, detach_reset), h
    h = charge(kind, x, v, tau_or_w, decay_input, v_reset)
    spike = sg(h - v_threshold)
    return spike, voltage_reset(h, spike, v_threshold, v_reset, detach_reset), h


def izhikevich_step(x, v, w, tau, a0, v_rest, v_c, tau_w, a, b, v_threshold, v_reset: Optional[float], sg: Callable,
                    detach_reset: bool):
    """(spike, v_next, w_next, h): functional/neuron.py:1514-1522."""
    v_charged = v + (x + a0 * (v - v_rest) * (v - v_c) - w) / tau
    w_next = w + (a * (v_charged - v_rest) - w) / tau_w
    spike = sg(v_charged - v_threshold)
    spike_d = spike.detach() if detach_reset else spike
    if v_reset is None:
        v_next = v_charged - spike_d * v_threshold
    else:
        v_next = (1.0 - spike_d) * v_charged + spike * v_reset
    return spike, v_next, w_next + b * spike, v_charged


def izhikevich_multi_step(x_seq, v_init, w_init, params, v_threshold: float, v_reset: Optional[float],
                          sg: Optional[Callable] = None, detach_reset: bool = False):
    """Step loop (base.py:594-607) over ``izhikevich_step``; ``params`` = (tau, a0, v_rest, v_c, tau_w, a, b).
    Returns (spike_seq, v_seq, w_seq, h_seq)."""
    sg = heaviside if sg is None else sg
    tau, a0, v_rest, v_c, tau_w, a, b = params
    v, w, out = v_init, w_init, ([], [], [], [])
    for t in range(x_seq.shape[0]):
        s, v, w, h = izhikevich_step(x_seq[t], v, w, tau, a0, v_rest, v_c, tau_w, a, b, v_threshold, v_reset, sg,
                                     detach_reset)
        for seq, value in zip(out, (s, v, w, h)):
            seq.append(value)
    return tuple(torch.stack(seq) for seq in out)


def activation_aware_if_step(x, v, v_threshold, v_offset, v_reset: Optional[float], sg: Callable, detach_reset: bool):
    """(spike, v_next, h): functional/neuron.py:577-584; v_threshold / v_offset are tensors broadcastable to x."""
    h = v + x
    spike = sg(h + v_offset - v_threshold)
    spike_d = spike.detach() if detach_reset else spike
    if v_reset is None:
        v_next = h - spike_d * v_threshold
    else:
        v_next = spike_d * v_reset + (1.0 - spike_d) * h
    return spike, v_next, h


def activation_aware_if_multi_step(x_seq, v_init, v_threshold, v_offset, channel_dim: int, v_reset: Optional[float]):
    """Step loop of neuron/integrate_and_fire.py:1125-1137 with the parameter broadcast of :879-895 (1-D parameters
    lie along ``channel_dim`` of one time step, cast to the input's dtype).  Returns (spike_seq, v_seq)."""
    def shaped(param):
        param = torch.as_tensor(param).to(x_seq.dtype)
        if param.dim() == 0:
            return param
        shape = [1] * (x_seq.dim() - 1)
        shape[channel_dim] = param.numel()
        return param.view(shape)

    th, off = shaped(v_threshold), shaped(v_offset)
    v, s_steps, v_steps = v_init, [], []
    for t in range(x_seq.shape[0]):
        s, v, _ = activation_aware_if_step(x_seq[t], v, th, off, v_reset, heaviside, False)
        s_steps.append(s)
        v_steps.append(v)
    return torch.stack(s_steps), torch.stack(v_steps)


# ------------------------------------------------------------------------------------------------
# sequences
# ------------------------------------------------------------------------------------------------


def multi_step(kind: str, x_seq: torch.Tensor, v_init: torch.Tensor, tau_or_w=None, decay_input: bool = True,
               v_threshold: float = 1.0, v_reset: Optional[float] = 0.0, sg: Optional[Callable] = None,
               detach_reset: bool = False):
    """Step loop + stack (base.py:594-607, neuron/base_node.py:449-464).

    Returns (spike_seq, v_seq, h_seq); state dtype follows ``x_seq`` as ``full_like`` makes it in
    ``neuron/base_node.py:474-475``.
    """
    sg = heaviside if sg is None else sg
    v = v_init
    s_steps, v_steps, h_steps = [], [], []
    for t in range(x_seq.shape[0]):
        s, v, h = step(kind, x_seq[t], v, tau_or_w, decay_input, v_threshold, v_reset, sg, detach_reset)
        s_steps.append(s)
        v_steps.append(v)
        h_steps.append(h)
    return torch.stack(s_steps), torch.stack(v_steps), torch.stack(h_steps)


def multi_step_mixed_precision(kind: str, x_seq: torch.Tensor, v_init: torch.Tensor, storage_dtype: torch.dtype,
                               k: float = 0.5, decay_input: bool = True, v_threshold: float = 1.0,
                               v_reset: Optional[float] = 0.0, torch_op_order: bool = True,
                               return_raw_h: bool = False):
    """fp32 state and arithmetic, storage-dtype inputs/outputs
    (test/activation_based/test_triton_neuron.py:212-247): inputs are quantised to the storage dtype,
    v is carried in fp32 un-rounded, stored v/h are rounded.  ``torch_op_order`` keeps the torch
    backend's expression order (what the HIP kernels use); False uses the test's
    ``v + k*(reset - v + x)`` order -- identical when v_reset is 0 or None.
    Returns fp32 tensors (spike_seq, v_seq, h_seq) holding storage-representable values; with
    ``return_raw_h`` a fourth tensor holds h before it was rounded for storage.
    """
    q = lambda t: t.to(storage_dtype).to(torch.float32)
    x_seq = q(x_seq)
    v = q(v_init)
    k = torch.tensor(k, dtype=torch.float32)
    reset_value = 0.0 if v_reset is None else v_reset
    s_seq = torch.empty_like(x_seq)
    v_seq = torch.empty_like(x_seq)
    h_seq = torch.empty_like(x_seq)
    raw_h_seq = torch.empty_like(x_seq)
    for t in range(x_seq.shape[0]):
        x = x_seq[t]
        if kind == "if":
            h = v + x
        elif torch_op_order:
            h = charge("plif_k", x, v, k, decay_input, v_reset)
        elif decay_input:
            h = v + k * (reset_value - v + x)
        else:
            h = v + k * (reset_value - v) + x
        s = ((h - v_threshold) >= 0).to(torch.float32)
        if v_reset is None:
            v = h - s * v_threshold
        else:
            v = s * reset_value + (1.0 - s) * h
        s_seq[t] = s
        v_seq[t] = q(v)
        h_seq[t] = q(h)
        raw_h_seq[t] = h
    if return_raw_h:
        return s_seq, v_seq, h_seq, raw_h_seq
    return s_seq, v_seq, h_seq


def forward_backward(kind: str, x_seq: torch.Tensor, v_init: torch.Tensor, grad_spike_seq: Optional[torch.Tensor],
                     grad_v_seq: Optional[torch.Tensor] = None, grad_v_last: Optional[torch.Tensor] = None,
                     tau_or_w=None, decay_input: bool = True, v_threshold: float = 1.0,
                     v_reset: Optional[float] = 0.0, sg_name: str = "atan", sg_alpha: float = 2.0,
                     detach_reset: bool = False, spiking: bool = True, sg: Optional[Callable] = None):
    """Forward with the surrogate, then autograd with the given upstream gradients.  ``sg`` overrides the
    surrogate named by ``sg_name`` (ILIF: ``multi_level_spike_count(D, window)``).

    Returns dict(spike_seq, v_seq, h_seq, grad_x, grad_v_init[, grad_p]) where grad_p is the
    gradient w.r.t. ``tau_or_w`` when that is a tensor (PLIF's ``w`` or ``k``).
    """
    x = x_seq.detach().clone().requires_grad_(True)
    v0 = v_init.detach().clone().requires_grad_(True)
    p = tau_or_w
    if isinstance(p, torch.Tensor):
        p = p.detach().clone().requires_grad_(True)
    s_seq, v_seq, h_seq = multi_step(kind, x, v0, p, decay_input, v_threshold, v_reset,
                                     surrogate(sg_name, sg_alpha, spiking) if sg is None else sg, detach_reset)
    outs, grads = [], []
    if grad_spike_seq is not None:
        outs.append(s_seq)
        grads.append(grad_spike_seq)
    if grad_v_seq is not None:
        outs.append(v_seq)
        grads.append(grad_v_seq)
    if grad_v_last is not None:
        outs.append(v_seq[-1])
        grads.append(grad_v_last)
    torch.autograd.backward(outs, grads)
    res = dict(spike_seq=s_seq.detach(), v_seq=v_seq.detach(), h_seq=h_seq.detach(),
               grad_x=x.grad if x.grad is not None else torch.zeros_like(x),
               grad_v_init=v0.grad if v0.grad is not None else torch.zeros_like(v0))
    if isinstance(p, torch.Tensor):
        res["grad_p"] = p.grad if p.grad is not None else torch.zeros_like(p)
    return res
