"""Functional state transitions of IF / LIF / PLIF neurons.

Two families, as in the reference's ``spikingjelly/activation_based/functional/neuron.py``:

* ``*_step`` / ``voltage_reset`` / ``lif_charge``: the torch-backend math, one step, pure
  (reference :173-228, :242-312, :797-933, :1215-1297);
* ``{if,lif,plif}_multi_step_hip``: whole sequences through the HIP kernels, same signature and
  return convention as the reference's ``*_multi_step_cupy`` / ``*_multi_step_triton``
  (:1889-2185, :2582-2849): ``(spike_seq, v_next, v_seq or None)``;
* ``{if,lif,plif}_step_hip``: one step through the same kernels (a sequence of length one), signature and
  return of the reference's ``*_step_cupy`` (:1709-1886): ``(spike, v_next)``;
* ``{if,lif,plif}_multi_step_hip_packed``: inference only, the spikes come back bit-packed
  (``bit_spike_compress`` layout) instead of as a dense tensor: ``(spike_bits, v_next, v_seq or None)``.
  It is the fused form of a kernel-backend neuron followed by the reference's ``BitSpikeCompressor``
  (``memopt/compress.py:332-385``); unpack with ``bit_spike_decompress(spike_bits, x_seq.shape, dtype)``.
"""

from __future__ import annotations

from typing import Callable, Optional

import torch

from ... import configure

SurrogateFunction = Callable[[torch.Tensor], torch.Tensor]

__all__ = [
    "voltage_reset",
    "if_step",
    "lif_charge",
    "lif_step",
    "plif_step",
    "qif_step",
    "eif_step",
    "izhikevich_step",
    "ilif_step",
    "stbif_step",
    "activation_aware_if_step",
    "if_multi_step_hip",
    "lif_multi_step_hip",
    "plif_multi_step_hip",
    "qif_multi_step_hip",
    "eif_multi_step_hip",
    "izhikevich_multi_step_hip",
    "ilif_multi_step_hip",
    "stbif_multi_step_hip",
    "stbif_single_step_hip",
    "activation_aware_if_multi_step_hip",
    "if_step_hip",
    "lif_step_hip",
    "plif_step_hip",
    "if_multi_step_hip_packed",
    "lif_multi_step_hip_packed",
    "plif_multi_step_hip_packed",
]


# ---- torch backend: one step --------------------------------------------------------------------
def voltage_reset(v: torch.Tensor, spike: torch.Tensor, v_threshold: float, v_reset: Optional[float],
                  detach_reset: bool) -> torch.Tensor:
    """Soft reset ``v - s*v_threshold`` when ``v_reset is None``, else hard reset
    ``s*v_reset + (1 - s)*v``; ``detach_reset`` cuts the gradient through ``s`` here only."""
    s = spike.detach() if detach_reset else spike
    if v_reset is None:
        return v - s * v_threshold
    return s * v_reset + (1.0 - s) * v


def if_step(x: torch.Tensor, v: torch.Tensor, v_threshold: float, v_reset: Optional[float],
            surrogate_function: SurrogateFunction, detach_reset: bool = False
            ) -> tuple[torch.Tensor, torch.Tensor]:
    """One IF step: ``h = v + x``, fire, reset.  Returns ``(spike, v_next)``."""
    h = v + x
    spike = surrogate_function(h - v_threshold)
    return spike, voltage_reset(h, spike, v_threshold, v_reset, detach_reset)


def lif_charge(x: torch.Tensor, v: torch.Tensor, tau: float, decay_input: bool,
               v_reset: Optional[float]) -> torch.Tensor:
    """LIF charge; ``v_reset=None`` counts as 0 here."""
    rest = 0.0 if v_reset is None else v_reset
    if decay_input:
        return v + (x - (v - rest)) / tau
    return v - (v - rest) / tau + x


def lif_step(x: torch.Tensor, v: torch.Tensor, tau: float, decay_input: bool, v_threshold: float,
             v_reset: Optional[float], surrogate_function: SurrogateFunction, detach_reset: bool = False
             ) -> tuple[torch.Tensor, torch.Tensor]:
    """One LIF step.  Returns ``(spike, v_next)``."""
    h = lif_charge(x, v, tau, decay_input, v_reset)
    spike = surrogate_function(h - v_threshold)
    return spike, voltage_reset(h, spike, v_threshold, v_reset, detach_reset)


def plif_step(x: torch.Tensor, v: torch.Tensor, w: torch.Tensor, decay_input: bool, v_threshold: float,
              v_reset: Optional[float], surrogate_function: SurrogateFunction, detach_reset: bool = False
              ) -> tuple[torch.Tensor, torch.Tensor]:
    """One parametric-LIF step with ``1/tau = sigmoid(w)``.  Returns ``(spike, v_next)``."""
    k = w.sigmoid()
    rest = 0.0 if v_reset is None else v_reset
    if decay_input:
        h = v + (x - (v - rest)) * k
    else:
        h = v - (v - rest) * k + x
    spike = surrogate_function(h - v_threshold)
    return spike, voltage_reset(h, spike, v_threshold, v_reset, detach_reset)


def qif_step(x: torch.Tensor, v: torch.Tensor, tau: float, a0: float, v_rest: float, v_c: float, v_threshold: float,
             v_reset: Optional[float], surrogate_function: SurrogateFunction, detach_reset: bool = False
             ) -> tuple[torch.Tensor, torch.Tensor]:
    """One quadratic integrate-and-fire step (reference :315-399): ``h = v + (x + a0 (v - v_rest)(v - v_c)) / tau``."""
    h = v + (x + a0 * (v - v_rest) * (v - v_c)) / tau
    spike = surrogate_function(h - v_threshold)
    return spike, voltage_reset(h, spike, v_threshold, v_reset, detach_reset)


def eif_step(x: torch.Tensor, v: torch.Tensor, tau: float, delta_t: float, theta_rh: float, v_rest: float,
             v_threshold: float, v_reset: Optional[float], surrogate_function: SurrogateFunction,
             detach_reset: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """One exponential integrate-and-fire step (reference :402-487):
    ``h = v + (x + v_rest - v + delta_t exp((v - theta_rh) / delta_t)) / tau``."""
    h = v + (x + v_rest - v + delta_t * torch.exp((v - theta_rh) / delta_t)) / tau
    spike = surrogate_function(h - v_threshold)
    return spike, voltage_reset(h, spike, v_threshold, v_reset, detach_reset)


def izhikevich_step(x: torch.Tensor, v: torch.Tensor, w: torch.Tensor, tau: float, a0: float, v_rest: float, v_c: float,
                    tau_w: float, a: float, b: float, v_threshold: float, v_reset: Optional[float],
                    surrogate_function: SurrogateFunction, detach_reset: bool = False
                    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """One Izhikevich step (reference :1412-1522): a quadratic membrane ``v`` with an adaptation current ``w`` that
    follows the membrane (``a``, ``tau_w``) and jumps by ``b`` at a spike.  Returns ``(spike, v_next, w_next)``.  In the
    hard reset the ``v_reset`` term carries the undetached spike, as in the reference."""
    h = v + (x + a0 * (v - v_rest) * (v - v_c) - w) / tau
    w_next = w + (a * (h - v_rest) - w) / tau_w
    spike = surrogate_function(h - v_threshold)
    s = spike.detach() if detach_reset else spike
    if v_reset is None:
        v_next = h - s * v_threshold
    else:
        v_next = (1.0 - s) * h + spike * v_reset
    return spike, v_next, w_next + b * spike


def ilif_step(x: torch.Tensor, v: torch.Tensor, tau: float, v_threshold: float,
              surrogate_function: SurrogateFunction, detach_reset: bool = False
              ) -> tuple[torch.Tensor, torch.Tensor]:
    """One integer-valued LIF step (reference :1030-1099): the LIF charge without input decay and with
    ``v_reset=None``, a multi-level count fired from ``h / v_threshold``, a soft reset by ``count * v_threshold``.
    Returns ``(count, v_next)``."""
    h = lif_charge(x, v, tau, False, None)
    count = surrogate_function(h / v_threshold)
    return count, voltage_reset(h, count, v_threshold, None, detach_reset)


def stbif_step(x: torch.Tensor, q: torch.Tensor, acc_q: torch.Tensor, q_threshold: torch.Tensor,
               pos_max: torch.Tensor, neg_min: torch.Tensor
               ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """One step of SpikeZIP's signed ternary neuron (reference :3144-3247), inference semantics: the input in units
    of the quantiser scale joins the residual ``q``; a unit is released upwards when ``q >= 1`` and the released
    total ``acc_q`` is below ``pos_max``, downwards when ``q < 0`` and it is above ``neg_min``.
    Returns ``(out, q_next, acc_q_next, cur_output_next)`` with ``out = cur_output_next * q_threshold``."""
    q_threshold, pos_max, neg_min = q_threshold.to(x), pos_max.to(x), neg_min.to(x)
    q_next = q + (x / q_threshold).detach()
    acc_next = torch.round(acc_q)
    up = (q_next - 1 >= 0) & (acc_next < pos_max)
    down = (q_next < 0) & (acc_next > neg_min)
    cur = up.to(x.dtype) - down.to(x.dtype)
    acc_next = acc_next + cur
    q_next = torch.where(up, q_next - 1, q_next)
    q_next = torch.where(down, q_next + 1, q_next)
    return cur * q_threshold, q_next, acc_next, cur


def activation_aware_if_step(x: torch.Tensor, v: torch.Tensor, v_threshold: torch.Tensor, v_offset: torch.Tensor,
                             v_reset: Optional[float], surrogate_function: SurrogateFunction,
                             detach_reset: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """One step of an IF neuron that fires on ``h + v_offset >= v_threshold`` (reference :502-584); both parameters
    are already broadcastable to ``x``.  Returns ``(spike, v_next)``."""
    h = v + x
    spike = surrogate_function(h + v_offset - v_threshold)
    s = spike.detach() if detach_reset else spike
    if v_reset is None:
        return spike, h - s * v_threshold
    return spike, s * v_reset + (1.0 - s) * h


# ---- hip backend: whole sequence ----------------------------------------------------------------
def _hip_mode_flags(x_seq: torch.Tensor) -> int:
    from ..hip_kernel import library as L

    flags = 0
    if x_seq.dtype != torch.float32:
        mode = configure.hip_half_precision_mode
        if mode == "fp32_state":
            flags |= L.FLAG_FP32_STATE
        elif mode != "torch":
            raise ValueError(f"configure.hip_half_precision_mode must be 'torch' or 'fp32_state', got {mode!r}")
    if configure.hip_lif_reciprocal_tau:
        flags |= L.FLAG_RECIPROCAL_TAU
    if configure.hip_plif_atomic_reduce:
        flags |= L.FLAG_ATOMIC_REDUCE
    return flags


@torch.compiler.assume_constant_result
def _replay_limits(dtype: torch.dtype, flags: int) -> tuple[int, int]:
    """``(vector width, longest sequence)`` of the library's replay policy for one dtype and mode: replay is preferred
    for ``[T, N]`` when ``N`` is a multiple of the width and ``T`` does not exceed the length.  The policy itself lives
    in the library (``sjhip_recompute_preferred``, monotone in ``T``); it is probed once per ``(dtype, flags)`` and the
    answer is a constant of any traced graph, so the shape test below is plain integer arithmetic a tracing compiler
    can follow, also with symbolic shapes."""
    key = (dtype, flags & _REPLAY_POLICY_FLAGS)
    if key not in _replay_limits_cache:
        from ..hip_kernel import library as L

        width = next((n for n in (1, 2, 4, 8, 16) if L.recompute_preferred(dtype, 1, n, key[1])), 0)
        steps = 0
        while width and steps < 4096 and L.recompute_preferred(dtype, steps + 1, width, key[1]):
            steps += 1
        _replay_limits_cache[key] = (width, steps)
    return _replay_limits_cache[key]


_replay_limits_cache: dict = {}
_REPLAY_POLICY_FLAGS = 0x10  # FLAG_FP32_STATE: the only flag the policy depends on


def _hip_recompute(x2: torch.Tensor) -> bool:
    """Replay the forward inside the backward kernel instead of saving h_seq, when the shape allows and the
    sequence is short enough for the replay to pay (its LDS footprint grows with T)."""
    if not configure.hip_backward_recompute:
        return False
    width, steps = _replay_limits(x2.dtype, _hip_mode_flags(x2))
    return width > 0 and x2.shape[1] % width == 0 and x2.shape[0] <= steps


def _use_eager_entry() -> bool:
    """The direct ``autograd.Function`` entry serves ordinary eager calls; a tracing compiler needs the operators
    (schema, fake kernels)."""
    return not torch.compiler.is_compiling()


def _needs_grad(*tensors: torch.Tensor) -> bool:
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


def _finish(x_seq: torch.Tensor, spike_seq: torch.Tensor, v_seq: torch.Tensor, v_last: torch.Tensor,
            store_v_seq: bool) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    spike_seq = spike_seq.reshape(x_seq.shape)
    v_last = v_last.reshape(x_seq.shape[1:])
    return spike_seq, v_last, (v_seq.reshape(x_seq.shape) if store_v_seq else None)


def if_multi_step_hip(x_seq: torch.Tensor, v: torch.Tensor, v_threshold: float, v_reset: Optional[float],
                      surrogate_function: SurrogateFunction, detach_reset: bool = False,
                      store_v_seq: bool = False
                      ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Multi-step IF on the hip backend.  ``x_seq`` is ``[T, *]``, ``v`` has the shape of ``x_seq[0]``."""
    from ..hip_kernel import library as L
    from ..hip_kernel import neuron_kernel as K
    from ..hip_kernel.surrogate_registry import resolve_sg_hip_id_and_alpha

    soft = v_reset is None
    vr = 0.0 if soft else float(v_reset)
    flags = _hip_mode_flags(x_seq)
    x2, v1 = x_seq.flatten(1), v.flatten()
    need_grad = _needs_grad(x_seq, v)
    sg_id, sg_alpha = resolve_sg_hip_id_and_alpha(surrogate_function) if need_grad else (0, 0.0)
    if _use_eager_entry():
        s, v_seq, v_last = K.eager_multistep(L.NEURON_IF, x2, v1, None, 0.0, v_threshold, vr,
                                             K._flags(soft, detach_reset, False, flags), sg_id, sg_alpha, store_v_seq,
                                             need_grad and _hip_recompute(x2), need_grad)
    elif need_grad:
        s, v_seq, v_last, _ = K.hip_multistep_if_forward(x2, v1, v_threshold, vr, soft, detach_reset, sg_id,
                                                         sg_alpha, store_v_seq, flags, _hip_recompute(x2))
    else:
        s, v_seq, v_last = K.hip_multistep_if_inference(x2, v1, v_threshold, vr, soft, store_v_seq, flags)
    return _finish(x_seq, s, v_seq, v_last, store_v_seq)


def lif_multi_step_hip(x_seq: torch.Tensor, v: torch.Tensor, tau: float, decay_input: bool,
                       v_threshold: float, v_reset: Optional[float], surrogate_function: SurrogateFunction,
                       detach_reset: bool = False, store_v_seq: bool = False
                       ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Multi-step LIF on the hip backend."""
    from ..hip_kernel import library as L
    from ..hip_kernel import neuron_kernel as K
    from ..hip_kernel.surrogate_registry import resolve_sg_hip_id_and_alpha

    soft = v_reset is None
    vr = 0.0 if soft else float(v_reset)
    flags = _hip_mode_flags(x_seq)
    x2, v1 = x_seq.flatten(1), v.flatten()
    need_grad = _needs_grad(x_seq, v)
    sg_id, sg_alpha = resolve_sg_hip_id_and_alpha(surrogate_function) if need_grad else (0, 0.0)
    if _use_eager_entry():
        s, v_seq, v_last = K.eager_multistep(L.NEURON_LIF, x2, v1, None, float(tau), v_threshold, vr,
                                             K._flags(soft, detach_reset, decay_input, flags), sg_id, sg_alpha,
                                             store_v_seq, need_grad and _hip_recompute(x2), need_grad)
    elif need_grad:
        s, v_seq, v_last, _ = K.hip_multistep_lif_forward(x2, v1, v_threshold, vr, soft, detach_reset,
                                                          float(tau), decay_input, sg_id, sg_alpha,
                                                          store_v_seq, flags, _hip_recompute(x2))
    else:
        s, v_seq, v_last = K.hip_multistep_lif_inference(x2, v1, v_threshold, vr, soft, float(tau),
                                                         decay_input, store_v_seq, flags)
    return _finish(x_seq, s, v_seq, v_last, store_v_seq)


def plif_multi_step_hip(x_seq: torch.Tensor, v: torch.Tensor, w: torch.Tensor, decay_input: bool,
                        v_threshold: float, v_reset: Optional[float], surrogate_function: SurrogateFunction,
                        detach_reset: bool = False, store_v_seq: bool = False
                        ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Multi-step parametric LIF on the hip backend.  ``w`` is the pre-sigmoid parameter; the
    sigmoid stays outside the operator so autograd supplies ``dk/dw`` (reference :2173-2182)."""
    from ..hip_kernel import library as L
    from ..hip_kernel import neuron_kernel as K
    from ..hip_kernel.surrogate_registry import resolve_sg_hip_id_and_alpha

    soft = v_reset is None
    vr = 0.0 if soft else float(v_reset)
    flags = _hip_mode_flags(x_seq)
    x2, v1 = x_seq.flatten(1), v.flatten()
    k = w.sigmoid().to(device=x_seq.device, dtype=torch.float32)
    need_grad = _needs_grad(x_seq, v, w)
    sg_id, sg_alpha = resolve_sg_hip_id_and_alpha(surrogate_function) if need_grad else (0, 0.0)
    if _use_eager_entry():
        s, v_seq, v_last = K.eager_multistep(L.NEURON_PLIF, x2, v1, k, 0.0, v_threshold, vr,
                                             K._flags(soft, detach_reset, decay_input, flags), sg_id, sg_alpha,
                                             store_v_seq, need_grad and _hip_recompute(x2), need_grad)
    elif need_grad:
        s, v_seq, v_last, _ = K.hip_multistep_plif_forward(x2, v1, k, v_threshold, vr, soft, detach_reset,
                                                           decay_input, sg_id, sg_alpha, store_v_seq, flags,
                                                           _hip_recompute(x2))
    else:
        s, v_seq, v_last = K.hip_multistep_plif_inference(x2, v1, k, v_threshold, vr, soft, decay_input,
                                                          store_v_seq, flags)
    return _finish(x_seq, s, v_seq, v_last, store_v_seq)


def qif_multi_step_hip(x_seq: torch.Tensor, v: torch.Tensor, tau: float, v_threshold: float, v_reset: Optional[float],
                       v_rest: float, v_c: float, a0: float, detach_reset: bool,
                       surrogate_function: SurrogateFunction, store_v_seq: bool = False
                       ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Multi-step QIF on the hip backend; argument order of the reference's ``qif_multi_step_cupy`` (:2188-2200)."""
    from ..hip_kernel import library as L
    from ..hip_kernel import neuron_kernel as K
    from ..hip_kernel.surrogate_registry import resolve_sg_hip_id_and_alpha

    soft = v_reset is None
    vr = 0.0 if soft else float(v_reset)
    flags = _hip_mode_flags(x_seq)
    x2, v1 = x_seq.flatten(1), v.flatten()
    need_grad = _needs_grad(x_seq, v)
    sg_id, sg_alpha = resolve_sg_hip_id_and_alpha(surrogate_function) if need_grad else (0, 0.0)
    if _use_eager_entry():
        s, v_seq, v_last = K.eager_multistep(L.NEURON_QIF, x2, v1, None, float(tau), v_threshold, vr,
                                             K._flags(soft, detach_reset, True, flags), sg_id, sg_alpha, store_v_seq,
                                             need_grad and _hip_recompute(x2), need_grad,
                                             qif=(float(v_rest), float(v_c), float(a0)))
    elif need_grad:
        s, v_seq, v_last, _ = K.hip_multistep_qif_forward(x2, v1, v_threshold, vr, soft, detach_reset, float(tau),
                                                          float(v_rest), float(v_c), float(a0), sg_id, sg_alpha,
                                                          store_v_seq, flags, _hip_recompute(x2))
    else:
        s, v_seq, v_last = K.hip_multistep_qif_inference(x2, v1, v_threshold, vr, soft, float(tau), float(v_rest),
                                                         float(v_c), float(a0), store_v_seq, flags)
    return _finish(x_seq, s, v_seq, v_last, store_v_seq)


def eif_multi_step_hip(x_seq: torch.Tensor, v: torch.Tensor, tau: float, v_threshold: float, v_reset: Optional[float],
                       v_rest: float, theta_rh: float, delta_t: float, detach_reset: bool,
                       surrogate_function: SurrogateFunction, store_v_seq: bool = False
                       ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Multi-step EIF on the hip backend; argument order of the reference's ``eif_multi_step_cupy`` (:2296-2308)."""
    from ..hip_kernel import library as L
    from ..hip_kernel import neuron_kernel as K
    from ..hip_kernel.surrogate_registry import resolve_sg_hip_id_and_alpha

    soft = v_reset is None
    vr = 0.0 if soft else float(v_reset)
    flags = _hip_mode_flags(x_seq)
    x2, v1 = x_seq.flatten(1), v.flatten()
    need_grad = _needs_grad(x_seq, v)
    sg_id, sg_alpha = resolve_sg_hip_id_and_alpha(surrogate_function) if need_grad else (0, 0.0)
    if _use_eager_entry():
        s, v_seq, v_last = K.eager_multistep(L.NEURON_EIF, x2, v1, None, float(tau), v_threshold, vr,
                                             K._flags(soft, detach_reset, True, flags), sg_id, sg_alpha, store_v_seq,
                                             need_grad and _hip_recompute(x2), need_grad,
                                             qif=(float(v_rest), float(theta_rh), float(delta_t)))
    elif need_grad:
        s, v_seq, v_last, _ = K.hip_multistep_eif_forward(x2, v1, v_threshold, vr, soft, detach_reset, float(tau),
                                                          float(v_rest), float(theta_rh), float(delta_t), sg_id, sg_alpha,
                                                          store_v_seq, flags, _hip_recompute(x2))
    else:
        s, v_seq, v_last = K.hip_multistep_eif_inference(x2, v1, v_threshold, vr, soft, float(tau), float(v_rest),
                                                         float(theta_rh), float(delta_t), store_v_seq, flags)
    return _finish(x_seq, s, v_seq, v_last, store_v_seq)


def izhikevich_multi_step_hip(x_seq: torch.Tensor, v: torch.Tensor, w: torch.Tensor, tau: float, v_threshold: float,
                              v_reset: Optional[float], v_rest: float, a: float, b: float, tau_w: float, v_c: float,
                              a0: float, detach_reset: bool, surrogate_function: SurrogateFunction,
                              store_state_seq: bool = False, store_w_seq: Optional[bool] = None
                              ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, Optional[torch.Tensor],
                                         Optional[torch.Tensor]]:
    """Multi-step Izhikevich on the hip backend; arguments and return ``(spike_seq, v_next, w_next, v_seq | None,
    w_seq | None)`` of the reference's ``izhikevich_multi_step_cupy`` (:2404-2530).  ``store_w_seq=False`` with
    ``store_state_seq=True`` keeps only ``v_seq`` (what a node with ``store_v_seq`` needs) and saves the other write."""
    from ..hip_kernel import izhikevich_kernel as IK
    from ..hip_kernel.surrogate_registry import resolve_sg_hip_id_and_alpha

    soft = v_reset is None
    need_grad = _needs_grad(x_seq, v, w)
    sg_id, sg_alpha = resolve_sg_hip_id_and_alpha(surrogate_function) if need_grad else (0, 0.0)
    scalars = [float(tau), float(v_threshold), 0.0 if soft else float(v_reset), float(v_rest), float(v_c), float(a0),
               float(tau_w), float(a), float(b)]
    keep_w = store_state_seq if store_w_seq is None else bool(store_w_seq)
    x2 = x_seq.flatten(1)
    replay = need_grad and _hip_recompute(x2)
    s, v_seq, w_seq, v_last, w_last, _ = IK.hip_multistep_izhikevich_forward(
        x2, v.flatten(), w.flatten(), scalars, soft, detach_reset, sg_id, sg_alpha, store_state_seq, keep_w,
        need_grad and not replay, _hip_mode_flags(x_seq), replay)
    state = x_seq.shape[1:]
    return (s.reshape(x_seq.shape), v_last.reshape(state), w_last.reshape(state),
            v_seq.reshape(x_seq.shape) if store_state_seq else None, w_seq.reshape(x_seq.shape) if keep_w else None)


def ilif_multi_step_hip(x_seq: torch.Tensor, v: torch.Tensor, tau: float, v_threshold: float,
                        surrogate_function: SurrogateFunction, detach_reset: bool = False,
                        store_v_seq: bool = False
                        ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Multi-step integer-valued LIF on the hip backend; ``surrogate_function`` must be a spiking
    ``MultiLevelSpikeCount`` (its ``max_spike_count`` and gradient window go to the kernel, as the reference's
    Triton path passes them, ``neuron/ilif.py:343-353``).  ``spike_seq`` holds the counts."""
    from .. import surrogate
    from ..hip_kernel import library as L
    from ..hip_kernel import neuron_kernel as K

    if not isinstance(surrogate_function, surrogate.MultiLevelSpikeCount) or not surrogate_function.spiking:
        raise ValueError("surrogate_function must be a spiking MultiLevelSpikeCount.")
    levels = int(surrogate_function.max_spike_count)
    flags = _hip_mode_flags(x_seq)
    x2, v1 = x_seq.flatten(1), v.flatten()
    need_grad = _needs_grad(x_seq, v)
    if _use_eager_entry():
        s, v_seq, v_last = K.eager_multistep(
            L.NEURON_ILIF, x2, v1, None, float(tau), float(v_threshold), 0.0, K._flags(True, detach_reset, False, flags),
            L.SG_MULTI_LEVEL, 0.0, store_v_seq, need_grad and _hip_recompute(x2), need_grad,
            levels=(float(levels), float(surrogate_function.grad_min), float(surrogate_function.grad_max)))
    elif need_grad:
        s, v_seq, v_last, _ = K.hip_multistep_ilif_forward(
            x2, v1, float(tau), float(v_threshold), levels, float(surrogate_function.grad_min),
            float(surrogate_function.grad_max), detach_reset, store_v_seq, flags, _hip_recompute(x2))
    else:
        s, v_seq, v_last = K.hip_multistep_ilif_inference(x2, v1, float(tau), float(v_threshold), levels,
                                                          store_v_seq, flags)
    return _finish(x_seq, s, v_seq, v_last, store_v_seq)


@torch.no_grad()
def stbif_multi_step_hip(x_seq: torch.Tensor, q: torch.Tensor, acc_q: torch.Tensor, q_threshold: torch.Tensor,
                         pos_max: torch.Tensor, neg_min: torch.Tensor
                         ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Multi-step ST-BIF on the hip backend (inference only, like the reference's kernels).  Returns
    ``(out_seq, q_next, acc_q_next, cur_output, work_flag)``, the tuple of the reference's
    ``triton_kernel.neuron_kernel.stbif.multi_step_stbif`` (:337-399); ``work_flag`` is an int32 device scalar,
    non-zero when any input or output was non-zero."""
    from ..hip_kernel import stbif_kernel

    flags = _hip_mode_flags(x_seq)
    state_shape = x_seq.shape[1:]
    out, q2, acc2, cur, work = stbif_kernel.hip_multistep_stbif(x_seq.flatten(1), q.flatten(), acc_q.flatten(),
                                                                q_threshold, pos_max, neg_min, flags)
    return out.reshape(x_seq.shape), q2.reshape(state_shape), acc2.reshape(state_shape), cur.reshape(state_shape), work


def stbif_single_step_hip(x: torch.Tensor, q: torch.Tensor, acc_q: torch.Tensor, q_threshold: torch.Tensor,
                          pos_max: torch.Tensor, neg_min: torch.Tensor
                          ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """One ST-BIF step on the hip backend; return convention of the reference's ``stbif_single_step_triton``
    (:3250-3327)."""
    out, q2, acc2, cur, work = stbif_multi_step_hip(x.unsqueeze(0), q, acc_q, q_threshold, pos_max, neg_min)
    return out[0], q2, acc2, cur, work


@torch.no_grad()
def activation_aware_if_multi_step_hip(x_seq: torch.Tensor, v: torch.Tensor, v_threshold: torch.Tensor,
                                       v_offset: torch.Tensor, channel_size: int, inner_size: int,
                                       v_reset: Optional[float], store_v_seq: bool = False
                                       ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Multi-step activation-aware IF on the hip backend, inference only; signature and return of the reference's
    ``activation_aware_if_multi_step_triton`` (:587-660).  ``v_threshold`` / ``v_offset`` are scalars or hold
    ``channel_size`` values; channel ``(n // inner_size) % channel_size`` belongs to element ``n`` of a flattened
    step."""
    from ..hip_kernel import aaif_kernel

    soft = v_reset is None
    s, v_seq, v_last = aaif_kernel.hip_multistep_activation_aware_if(
        x_seq.flatten(1), v.flatten(), v_threshold, v_offset, int(channel_size), int(inner_size),
        0.0 if soft else float(v_reset), soft, store_v_seq, _hip_mode_flags(x_seq))
    return _finish(x_seq, s, v_seq, v_last, store_v_seq)


# ---- hip backend: one step (step_mode='s') --------------------------------------------------------
def if_step_hip(x: torch.Tensor, v: torch.Tensor, v_threshold: float, v_reset: Optional[float],
                surrogate_function: SurrogateFunction, detach_reset: bool = False
                ) -> tuple[torch.Tensor, torch.Tensor]:
    """One IF step on the hip backend: the multi-step kernel on a sequence of length one."""
    spike_seq, v_next, _ = if_multi_step_hip(x.unsqueeze(0), v, v_threshold, v_reset, surrogate_function,
                                             detach_reset, False)
    return spike_seq[0], v_next


def lif_step_hip(x: torch.Tensor, v: torch.Tensor, tau: float, decay_input: bool, v_threshold: float,
                 v_reset: Optional[float], surrogate_function: SurrogateFunction, detach_reset: bool = False
                 ) -> tuple[torch.Tensor, torch.Tensor]:
    """One LIF step on the hip backend."""
    spike_seq, v_next, _ = lif_multi_step_hip(x.unsqueeze(0), v, tau, decay_input, v_threshold, v_reset,
                                              surrogate_function, detach_reset, False)
    return spike_seq[0], v_next


def plif_step_hip(x: torch.Tensor, v: torch.Tensor, w: torch.Tensor, decay_input: bool, v_threshold: float,
                  v_reset: Optional[float], surrogate_function: SurrogateFunction, detach_reset: bool = False
                  ) -> tuple[torch.Tensor, torch.Tensor]:
    """One parametric-LIF step on the hip backend."""
    spike_seq, v_next, _ = plif_multi_step_hip(x.unsqueeze(0), v, w, decay_input, v_threshold, v_reset,
                                               surrogate_function, detach_reset, False)
    return spike_seq[0], v_next


# ---- hip backend: whole sequence, bit-packed spikes (inference) -----------------------------------
def _finish_packed(x_seq: torch.Tensor, out, store_v_seq: bool
                   ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    bits, v_seq, v_last = out
    return bits, v_last.reshape(x_seq.shape[1:]), (v_seq.reshape(x_seq.shape) if store_v_seq else None)


def _packed_by_two_kernels(dense_out) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """N % 8 != 0: a time step does not start on a byte, so the dense kernel runs and its spikes are packed."""
    from ..hip_kernel.compress import bit_spike_compress

    s, v_seq, v_last = dense_out
    return bit_spike_compress(s), v_seq, v_last


@torch.no_grad()
def if_multi_step_hip_packed(x_seq: torch.Tensor, v: torch.Tensor, v_threshold: float, v_reset: Optional[float],
                             store_v_seq: bool = False
                             ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Multi-step IF inference on the hip backend with bit-packed spike output."""
    from ..hip_kernel import neuron_kernel as K

    soft = v_reset is None
    vr = 0.0 if soft else float(v_reset)
    flags = _hip_mode_flags(x_seq)
    x2, v1 = x_seq.flatten(1), v.flatten()
    if K.packed_supported(x2.shape[1]):
        out = K.hip_multistep_if_inference_packed(x2, v1, v_threshold, vr, soft, store_v_seq, flags)
    else:
        out = _packed_by_two_kernels(K.hip_multistep_if_inference(x2, v1, v_threshold, vr, soft, store_v_seq, flags))
    return _finish_packed(x_seq, out, store_v_seq)


@torch.no_grad()
def lif_multi_step_hip_packed(x_seq: torch.Tensor, v: torch.Tensor, tau: float, decay_input: bool,
                              v_threshold: float, v_reset: Optional[float], store_v_seq: bool = False
                              ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Multi-step LIF inference on the hip backend with bit-packed spike output."""
    from ..hip_kernel import neuron_kernel as K

    soft = v_reset is None
    vr = 0.0 if soft else float(v_reset)
    flags = _hip_mode_flags(x_seq)
    x2, v1 = x_seq.flatten(1), v.flatten()
    if K.packed_supported(x2.shape[1]):
        out = K.hip_multistep_lif_inference_packed(x2, v1, v_threshold, vr, soft, float(tau), decay_input,
                                                   store_v_seq, flags)
    else:
        out = _packed_by_two_kernels(K.hip_multistep_lif_inference(x2, v1, v_threshold, vr, soft, float(tau),
                                                                   decay_input, store_v_seq, flags))
    return _finish_packed(x_seq, out, store_v_seq)


@torch.no_grad()
def plif_multi_step_hip_packed(x_seq: torch.Tensor, v: torch.Tensor, w: torch.Tensor, decay_input: bool,
                               v_threshold: float, v_reset: Optional[float], store_v_seq: bool = False
                               ) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """Multi-step parametric-LIF inference on the hip backend with bit-packed spike output."""
    from ..hip_kernel import neuron_kernel as K

    soft = v_reset is None
    vr = 0.0 if soft else float(v_reset)
    flags = _hip_mode_flags(x_seq)
    x2, v1 = x_seq.flatten(1), v.flatten()
    k = w.sigmoid().to(device=x_seq.device, dtype=torch.float32)
    if K.packed_supported(x2.shape[1]):
        out = K.hip_multistep_plif_inference_packed(x2, v1, k, v_threshold, vr, soft, decay_input, store_v_seq, flags)
    else:
        out = _packed_by_two_kernels(K.hip_multistep_plif_inference(x2, v1, k, v_threshold, vr, soft, decay_input,
                                                                    store_v_seq, flags))
    return _finish_packed(x_seq, out, store_v_seq)
