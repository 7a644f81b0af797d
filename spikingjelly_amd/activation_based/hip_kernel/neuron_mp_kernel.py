"""Mixed-precision multi-step IF / LIF / PLIF: storage dtype, compute dtype and spike dtype chosen separately.

Counterpart of the reference's experimental mixed-precision operators (``triton_kernel/neuron_kernel/lif.py:788-1150``,
``plif.py:720-1100``, ``integrate_and_fire.py:700-1050``; plan object ``neuron_kernel/utils.py:20-228``):

    multistep_{if,lif,plif}_mp(x_seq, v_init, [r_tau,] *, ..., storage_dtype, compute_dtype="fp32",
                               backward_compute_dtype="fp32", spike_dtype=torch.float32, save_intermediates=True,
                               detach_reset=False, surrogate_function=None) -> (s_seq, v_seq, h_seq | None)
    multistep_{if,lif,plif}_mp_with_plan(x_seq, v_init, [r_tau,] plan, *, ...)
    prepare_hip_neuron_execution_plan(neuron_type=..., device=..., storage_dtype=..., ...) -> HipNeuronExecutionPlan

``x_seq`` and ``v_init`` are rounded to ``storage_dtype``; the recurrence runs in fp32 on those values; ``v_seq`` and
``h_seq`` come back in the storage dtype, the spikes in ``spike_dtype``; gradients come back in the dtypes of the
inputs.  That is the recipe the reference checks its operators against (``test_triton_neuron.py:212-247``).

* ``float8_e4m3fn`` / ``float8_e5m2`` storage runs the 8-bit kernels (``sjhip_neuron_forward_mp`` /
  ``sjhip_neuron_backward_mp``: 1 B per stored element, 16 neurons per work-item).
* fp32 / fp16 / bf16 storage runs the ordinary kernels in their fp32-state mode; a different spike dtype is one cast.
* A 16-bit compute dtype equal to the storage dtype is the kernels' round-every-op mode.  Any other compute dtype
  (fp8 arithmetic, bf16 arithmetic on fp16 storage, ...) raises ``NotImplementedError``: the reference itself warns
  that those modes "may produce incorrect spike patterns" and keeps them for experiments.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional

import torch

from . import library as L
from . import neuron_kernel as K
from .surrogate_registry import resolve_sg_hip_id_and_alpha

__all__ = ["HipNeuronExecutionPlan", "prepare_hip_neuron_execution_plan", "normalize_storage_dtype",
           "normalize_compute_dtype_name", "is_fp8_dtype", "multistep_if_mp", "multistep_lif_mp", "multistep_plif_mp",
           "multistep_if_mp_with_plan", "multistep_lif_mp_with_plan", "multistep_plif_mp_with_plan",
           "hip_multistep_mp_forward", "hip_multistep_mp_backward"]

_STORAGE_ALIASES = {
    "fp32": torch.float32, "float32": torch.float32, "float": torch.float32,
    "fp16": torch.float16, "float16": torch.float16, "half": torch.float16,
    "bf16": torch.bfloat16, "bfloat16": torch.bfloat16,
    "float8_e4m3fn": torch.float8_e4m3fn, "fp8_e4m3fn": torch.float8_e4m3fn, "e4m3fn": torch.float8_e4m3fn,
    "float8_e5m2": torch.float8_e5m2, "fp8_e5m2": torch.float8_e5m2, "e5m2": torch.float8_e5m2,
}
_STORAGE_DTYPES = (torch.float32, torch.float16, torch.bfloat16, torch.float8_e4m3fn, torch.float8_e5m2)
_COMPUTE_NAMES = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16", torch.float8_e4m3fn: "fp8",
                  torch.float8_e5m2: "fp8"}
_F8_IDS = {torch.float8_e4m3fn: L.DTYPE_F8E4M3, torch.float8_e5m2: L.DTYPE_F8E5M2}
_SPIKE_DTYPES = (torch.float32, torch.float16, torch.bfloat16)
_NEURONS = {"if": L.NEURON_IF, "lif": L.NEURON_LIF, "plif": L.NEURON_PLIF}


def is_fp8_dtype(dtype: torch.dtype) -> bool:
    return dtype in _F8_IDS


def normalize_storage_dtype(storage_dtype) -> torch.dtype:
    """A torch dtype from a dtype or its name; ``"fp8"`` alone is refused as ambiguous (reference
    ``triton_utils.py:167-191``)."""
    if isinstance(storage_dtype, torch.dtype):
        dtype = storage_dtype
    elif isinstance(storage_dtype, str):
        key = storage_dtype.lower().replace("torch.", "")
        if key in ("fp8", "float8"):
            raise ValueError("storage_dtype='fp8' is ambiguous; use 'float8_e4m3fn' or 'float8_e5m2'.")
        if key not in _STORAGE_ALIASES:
            raise ValueError(f"Unsupported storage dtype: {storage_dtype!r}.")
        dtype = _STORAGE_ALIASES[key]
    else:
        raise ValueError(f"storage_dtype must be a string or torch.dtype, but got {type(storage_dtype).__name__}.")
    if dtype not in _STORAGE_DTYPES:
        raise ValueError(f"Unsupported storage dtype: {dtype}.")
    return dtype


def normalize_compute_dtype_name(compute_dtype) -> str:
    """``"fp32"``, ``"fp16"``, ``"bf16"`` or ``"fp8"`` from a name or a torch dtype."""
    if isinstance(compute_dtype, torch.dtype):
        if compute_dtype not in _COMPUTE_NAMES:
            raise ValueError(f"Unsupported compute dtype: {compute_dtype}.")
        return _COMPUTE_NAMES[compute_dtype]
    if isinstance(compute_dtype, str):
        key = compute_dtype.lower().replace("torch.", "")
        if key in ("fp8", "float8"):
            return "fp8"
        if key in _STORAGE_ALIASES:
            return _COMPUTE_NAMES[_STORAGE_ALIASES[key]]
    raise ValueError(f"Unsupported compute dtype: {compute_dtype!r}.")


def _normalize_device(device) -> torch.device:
    device = torch.device("cuda", device) if isinstance(device, int) else torch.device(device)
    if device.type == "cuda" and device.index is None:
        device = torch.device("cuda", torch.cuda.current_device() if torch.cuda.is_available() else 0)
    return device


@dataclass(frozen=True)
class HipNeuronExecutionPlan:
    """What a mixed-precision call resolves once: validated dtypes and the kernel route."""

    neuron_type: str
    device: torch.device
    storage_dtype: torch.dtype
    forward_compute_dtype_name: str
    backward_compute_dtype_name: str
    spike_dtype: torch.dtype
    save_intermediates: bool
    round_every_op: bool  # 16-bit storage computed in the storage dtype

    def matches(self, *, neuron_type: str, device, storage_dtype, forward_compute_dtype, backward_compute_dtype="fp32",
                spike_dtype: torch.dtype, save_intermediates: bool) -> bool:
        try:
            return (self.neuron_type == neuron_type and self.device == _normalize_device(device)
                    and self.storage_dtype == normalize_storage_dtype(storage_dtype)
                    and self.forward_compute_dtype_name == normalize_compute_dtype_name(forward_compute_dtype)
                    and self.backward_compute_dtype_name == normalize_compute_dtype_name(backward_compute_dtype)
                    and self.spike_dtype == spike_dtype and self.save_intermediates == save_intermediates)
        except (ValueError, RuntimeError, TypeError):
            return False


def prepare_hip_neuron_execution_plan(*, neuron_type: str, device, storage_dtype, forward_compute_dtype="fp32",
                                      backward_compute_dtype="fp32", spike_dtype: torch.dtype = torch.float32,
                                      save_intermediates: bool = True) -> HipNeuronExecutionPlan:
    if neuron_type not in _NEURONS:
        raise ValueError(f"neuron_type must be one of 'if', 'lif', or 'plif', but got {neuron_type!r}.")
    storage = normalize_storage_dtype(storage_dtype)
    forward_name = normalize_compute_dtype_name(forward_compute_dtype)
    try:
        backward_name = normalize_compute_dtype_name(backward_compute_dtype)
    except ValueError as e:
        raise ValueError(f"Invalid backward_compute_dtype: {e}") from e
    for label, name in (("compute_dtype", forward_name), ("backward_compute_dtype", backward_name)):
        if name == "fp8" and not is_fp8_dtype(storage):
            raise ValueError(f"{label}='fp8' requires an FP8 storage_dtype.")
    if spike_dtype not in _SPIKE_DTYPES:
        raise ValueError(f"spike_dtype must be torch.float32, torch.float16, or torch.bfloat16, but got {spike_dtype}.")
    if not isinstance(save_intermediates, bool):
        raise ValueError("save_intermediates must be bool.")
    device = _normalize_device(device)
    if device.type != "cuda":
        raise RuntimeError("hip neuron execution plan is unavailable: requires a ROCm device tensor.")
    storage_name = _COMPUTE_NAMES[storage]
    round_every_op = forward_name != "fp32" and forward_name == storage_name and not is_fp8_dtype(storage)
    if forward_name != "fp32" and not round_every_op:
        raise NotImplementedError(f"compute_dtype={forward_name!r} with storage {storage}: the hip kernels compute in fp32, "
                                  "or in a 16-bit storage dtype itself")
    if backward_name != "fp32":
        raise NotImplementedError(f"backward_compute_dtype={backward_name!r}: the hip backward computes in fp32")
    if is_fp8_dtype(storage):
        _check_fp8_capability(storage, device, neuron_type, save_intermediates)
    return HipNeuronExecutionPlan(neuron_type, device, storage, forward_name, backward_name, spike_dtype,
                                  save_intermediates, round_every_op)


def _check_fp8_capability(storage: torch.dtype, device: torch.device, neuron_type: str, with_backward: bool) -> None:
    """The reference's check at plan preparation (``triton_kernel/neuron_kernel/utils.py:99-152``): a forward (and, when
    intermediates are kept for it, a backward) that the device cannot run is refused here, with the probe's reason.
    The probes run once per dtype and device; nothing is probed while a HIP graph is being recorded."""
    from . import fp8_capability as C

    if C.probing() or not torch.cuda.is_available() or torch.cuda.is_current_stream_capturing():
        return  # (without a device there is nothing to ask; the operators refuse CPU tensors themselves)
    asks = [("forward", "compute_dtype", C.hip_fp8_neuron_capability)]
    if with_backward:
        asks.append(("backward", "backward_compute_dtype", C.hip_fp8_neuron_backward_capability))
    for pass_name, kw, ask in asks:
        answer = ask(storage, device, "fp32")
        if not answer.get("available", False):
            raise RuntimeError(f"hip FP8 {neuron_type.upper()} {pass_name} is unavailable for {storage} with "
                               f"{kw}='fp32': {answer.get('reason', 'unknown reason')}")


# ---- 8-bit storage: operators over the dedicated kernels -----------------------------------------------------------------

def _pad16(t: torch.Tensor) -> torch.Tensor:
    """Last dimension padded with zeros to a multiple of 16 elements, so that every row of every tensor of the call
    starts 16-byte aligned whatever its element size; the allocation itself 16-byte aligned."""
    n = t.shape[-1]
    if n % 16 == 0:
        return L.aligned16(t)
    out = t.new_zeros(t.shape[:-1] + ((n + 15) // 16 * 16,))
    out[..., :n] = t
    return out


def _mp_params(tau: float, v_th: float, v_reset: float, sg_alpha: float, sg_id: int, flags: int) -> L.NeuronParams:
    return K._params(tau, v_th, v_reset, sg_alpha, sg_id, flags)


@torch.library.custom_op("sj::hip_multistep_mp_forward", mutates_args=())
def hip_multistep_mp_forward(x_seq: torch.Tensor, v_init: torch.Tensor, k: Optional[torch.Tensor], neuron: int,
                             tau: float, decay_input: bool, v_th: float, v_reset: float, soft_reset: bool,
                             detach_reset: bool, sg_id: int, sg_alpha: float, storage_dtype: torch.dtype,
                             spike_dtype: torch.dtype, save_h: bool
                             ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``x_seq [T, N]``, ``v_init [N]`` of any float dtype -> ``(s_seq, v_seq, h_seq)``; 8-bit ``storage_dtype``."""
    L.require_device_tensor("x_seq", x_seq)
    L.require_device_tensor("v_init", v_init)
    if x_seq.dim() != 2 or v_init.shape != x_seq.shape[1:]:
        raise ValueError(f"x_seq must be [T, N] and v_init [N], got {tuple(x_seq.shape)} and {tuple(v_init.shape)}")
    T, N = x_seq.shape
    x8, v8 = _pad16(x_seq.to(storage_dtype)), _pad16(v_init.to(storage_dtype))
    Np = x8.shape[1]
    s = torch.empty((T, Np), dtype=spike_dtype, device=x_seq.device)
    v_seq = torch.empty((T, Np), dtype=storage_dtype, device=x_seq.device)
    h_seq = torch.empty((T, Np), dtype=storage_dtype, device=x_seq.device) if save_h else None
    k_keep, k_ptr = K._k_pointer(k, x_seq)
    params = _mp_params(tau, v_th, v_reset, 0.0, 0, K._flags(soft_reset, detach_reset, decay_input, 0))
    with torch.cuda.device(x_seq.device):
        rc = L.load().sjhip_neuron_forward_mp(neuron, _F8_IDS[storage_dtype], L.dtype_id(spike_dtype), ctypes.byref(params),
                                              T, Np, x8.data_ptr(), v8.data_ptr(), k_ptr, s.data_ptr(), v_seq.data_ptr(),
                                              None, L.ptr(h_seq), L.current_stream_ptr(x_seq.device))
    L.check(rc, "neuron_forward_mp")
    del k_keep
    crop = (lambda t: t) if Np == N else (lambda t: t[:, :N].contiguous())
    return crop(s), crop(v_seq), (crop(h_seq) if save_h else x_seq.new_empty((0,), dtype=storage_dtype))


@hip_multistep_mp_forward.register_fake
def _(x_seq, v_init, k, neuron, tau, decay_input, v_th, v_reset, soft_reset, detach_reset, sg_id, sg_alpha,
      storage_dtype, spike_dtype, save_h):
    return (x_seq.new_empty(x_seq.shape, dtype=spike_dtype), x_seq.new_empty(x_seq.shape, dtype=storage_dtype),
            x_seq.new_empty(x_seq.shape if save_h else (0,), dtype=storage_dtype))


@torch.library.custom_op("sj::hip_multistep_mp_backward", mutates_args=())
def hip_multistep_mp_backward(grad_s_seq: Optional[torch.Tensor], grad_v_seq: Optional[torch.Tensor],
                              h_seq: torch.Tensor, v_init: torch.Tensor, k: Optional[torch.Tensor], neuron: int,
                              tau: float, decay_input: bool, v_th: float, v_reset: float, soft_reset: bool,
                              detach_reset: bool, sg_id: int, sg_alpha: float, spike_dtype: torch.dtype,
                              grads_in_storage: bool = False) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """-> ``(grad_x_seq [T, N], grad_v_init [N], grad_k [] )``; ``grad_k`` (fp32) is zero unless PLIF.

    The first two are fp32, or, with ``grads_in_storage``, the 8-bit storage dtype: the kernel rounds its fp32 value
    once, which is what casting the fp32 result gives, and writes a quarter of the bytes (the reference allocates them
    in the dtypes of ``x_seq`` and ``v_init``, ``triton_kernel/neuron_kernel/lif.py:1115-1118``)."""
    L.require_device_tensor("h_seq", h_seq)
    storage_dtype = h_seq.dtype
    T, N = h_seq.shape
    h8 = _pad16(h_seq)
    Np = h8.shape[1]
    gs = _pad16((torch.zeros((T, N), dtype=spike_dtype, device=h_seq.device) if grad_s_seq is None
                 else grad_s_seq.to(spike_dtype)))
    gv = None if grad_v_seq is None else _pad16(grad_v_seq.to(storage_dtype))
    v8 = _pad16(v_init.to(storage_dtype))
    grad_dtype = storage_dtype if grads_in_storage else torch.float32
    grad_x = torch.empty((T, Np), dtype=grad_dtype, device=h_seq.device)
    grad_v_init = torch.empty((Np,), dtype=grad_dtype, device=h_seq.device)
    grad_k = torch.zeros((), dtype=torch.float32, device=h_seq.device)
    workspace = None
    if neuron == L.NEURON_PLIF:
        workspace = torch.empty((L.load().sjhip_plif_workspace_floats(L.DTYPE_F32, Np),), dtype=torch.float32,
                                device=h_seq.device)
    k_keep, k_ptr = K._k_pointer(k, h_seq)
    flags = K._flags(soft_reset, detach_reset, decay_input, 0) | (L.FLAG_GRAD_STORAGE if grads_in_storage else 0)
    params = _mp_params(tau, v_th, v_reset, sg_alpha, sg_id, flags)
    with torch.cuda.device(h_seq.device):
        rc = L.load().sjhip_neuron_backward_mp(neuron, _F8_IDS[storage_dtype], L.dtype_id(spike_dtype), ctypes.byref(params),
                                               T, Np, gs.data_ptr(), L.ptr(gv), None, h8.data_ptr(), v8.data_ptr(), k_ptr,
                                               grad_x.data_ptr(), grad_v_init.data_ptr(), grad_k.data_ptr(),
                                               L.ptr(workspace), L.current_stream_ptr(h_seq.device))
    L.check(rc, "neuron_backward_mp")
    del k_keep
    if Np != N:
        grad_x, grad_v_init = grad_x[:, :N].contiguous(), grad_v_init[:N].contiguous()
    return grad_x, grad_v_init, grad_k


@hip_multistep_mp_backward.register_fake
def _(grad_s_seq, grad_v_seq, h_seq, v_init, k, neuron, tau, decay_input, v_th, v_reset, soft_reset, detach_reset, sg_id,
      sg_alpha, spike_dtype, grads_in_storage=False):
    grad_dtype = h_seq.dtype if grads_in_storage else torch.float32
    return (h_seq.new_empty(h_seq.shape, dtype=grad_dtype), h_seq.new_empty(h_seq.shape[1:], dtype=grad_dtype),
            h_seq.new_empty((), dtype=torch.float32))


def _mp_setup(ctx, inputs, output):
    (x_seq, v_init, k, neuron, tau, decay_input, v_th, v_reset, soft_reset, detach_reset, sg_id, sg_alpha,
     storage_dtype, spike_dtype, save_h) = inputs
    if not save_h:
        raise RuntimeError("hip_multistep_mp_forward was called with save_h=False but needs a gradient")
    ctx.save_for_backward(output[2], v_init, k)
    ctx.dtypes = (x_seq.dtype, v_init.dtype, spike_dtype)
    ctx.scalars = (neuron, tau, decay_input, v_th, v_reset, soft_reset, detach_reset, sg_id, sg_alpha)
    ctx.set_materialize_grads(False)


def _mp_backward(ctx, grad_s_seq, grad_v_seq, grad_h_seq):
    del grad_h_seq
    h_seq, v_init, k = ctx.saved_tensors
    x_dtype, v_dtype, spike_dtype = ctx.dtypes
    in_storage = x_dtype == h_seq.dtype and v_dtype == h_seq.dtype  # otherwise fp32 results, cast below
    gx, gv0, gk = hip_multistep_mp_backward(grad_s_seq, grad_v_seq, h_seq, v_init, k, *ctx.scalars, spike_dtype, in_storage)
    grad_k = gk.to(k.dtype).reshape(k.shape) if (k is not None and ctx.needs_input_grad[2]) else None
    return (gx.to(x_dtype), gv0.to(v_dtype) if ctx.needs_input_grad[1] else None, grad_k) + (None,) * 12


torch.library.register_autograd("sj::hip_multistep_mp_forward", _mp_backward, setup_context=_mp_setup)


# ---- the public functions ----------------------------------------------------------------------------------------------

def _check_plan_inputs(x_seq: torch.Tensor, v_init: torch.Tensor, plan: HipNeuronExecutionPlan, name: str) -> None:
    if x_seq.device.type != "cuda" or v_init.device.type != "cuda":
        raise RuntimeError(f"Mixed-precision hip {name} forward requires ROCm device tensors.")
    if x_seq.device != v_init.device:
        raise RuntimeError("x_seq and v_init must be on the same device.")
    if v_init.shape != x_seq.shape[1:]:
        raise RuntimeError(f"v_init shape {v_init.shape} must match x_seq[0] shape {torch.Size(x_seq.shape[1:])}.")
    if _normalize_device(x_seq.device) != plan.device:
        raise RuntimeError(f"the plan was prepared for {plan.device}, the tensors are on {x_seq.device}.")


def _run(kind: str, x_seq: torch.Tensor, v_init: torch.Tensor, k: Optional[torch.Tensor], plan: HipNeuronExecutionPlan,
         tau: float, decay_input: bool, v_threshold: float, v_reset: Optional[float], detach_reset: bool,
         surrogate_function) -> tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    if plan.neuron_type != kind:
        raise ValueError(f"{kind.upper()} forward requires a {kind.upper()} plan, got {plan.neuron_type!r}.")
    _check_plan_inputs(x_seq, v_init, plan, kind.upper())
    soft = v_reset is None
    vr = 0.0 if soft else float(v_reset)
    tensors = (x_seq, v_init) if k is None else (x_seq, v_init, k)
    need_grad = torch.is_grad_enabled() and any(t.requires_grad for t in tensors)
    sg_id, sg_alpha = 0, 0.0
    if need_grad:
        from .. import surrogate

        sg_id, sg_alpha = resolve_sg_hip_id_and_alpha(surrogate.Sigmoid() if surrogate_function is None
                                                      else surrogate_function)
    shape = x_seq.shape
    x2, v1 = x_seq.flatten(1), v_init.flatten()
    neuron = _NEURONS[kind]
    if is_fp8_dtype(plan.storage_dtype):
        s, v_seq, h_seq = hip_multistep_mp_forward(x2, v1, k, neuron, float(tau), decay_input, float(v_threshold), vr, soft,
                                                   detach_reset, sg_id, sg_alpha, plan.storage_dtype, plan.spike_dtype,
                                                   need_grad or plan.save_intermediates)
    else:
        # the ordinary kernels on the rounded inputs: fp32 state (only stored values rounded) or every op rounded
        xs, vs = x2.to(plan.storage_dtype), v1.to(plan.storage_dtype)
        mode = 0 if (plan.round_every_op or plan.storage_dtype == torch.float32) else L.FLAG_FP32_STATE
        save_h = need_grad or plan.save_intermediates
        if kind == "if":
            out = (K.hip_multistep_if_forward(xs, vs, float(v_threshold), vr, soft, detach_reset, sg_id, sg_alpha, True,
                                              mode, False) if save_h
                   else K.hip_multistep_if_inference(xs, vs, float(v_threshold), vr, soft, True, mode))
        elif kind == "lif":
            out = (K.hip_multistep_lif_forward(xs, vs, float(v_threshold), vr, soft, detach_reset, float(tau), decay_input,
                                               sg_id, sg_alpha, True, mode, False) if save_h
                   else K.hip_multistep_lif_inference(xs, vs, float(v_threshold), vr, soft, float(tau), decay_input, True,
                                                      mode))
        else:
            out = (K.hip_multistep_plif_forward(xs, vs, k, float(v_threshold), vr, soft, detach_reset, decay_input, sg_id,
                                                sg_alpha, True, mode, False) if save_h
                   else K.hip_multistep_plif_inference(xs, vs, k, float(v_threshold), vr, soft, decay_input, True, mode))
        s, v_seq = out[0].to(plan.spike_dtype), out[1]
        h_seq = out[3] if save_h else None
    h_out = h_seq.reshape(shape) if (plan.save_intermediates and h_seq is not None and h_seq.numel()) else None
    return s.reshape(shape), v_seq.reshape(shape), h_out


def multistep_if_mp_with_plan(x_seq: torch.Tensor, v_init: torch.Tensor, plan: HipNeuronExecutionPlan, *,
                              v_threshold: float, v_reset: Optional[float], detach_reset: bool = False,
                              surrogate_function=None):
    return _run("if", x_seq, v_init, None, plan, 0.0, False, v_threshold, v_reset, detach_reset, surrogate_function)


def multistep_lif_mp_with_plan(x_seq: torch.Tensor, v_init: torch.Tensor, plan: HipNeuronExecutionPlan, *,
                               decay_input: bool, tau: float, v_threshold: float, v_reset: Optional[float],
                               detach_reset: bool = False, surrogate_function=None):
    return _run("lif", x_seq, v_init, None, plan, tau, decay_input, v_threshold, v_reset, detach_reset, surrogate_function)


def multistep_plif_mp_with_plan(x_seq: torch.Tensor, v_init: torch.Tensor, r_tau: torch.Tensor,
                                plan: HipNeuronExecutionPlan, *, decay_input: bool, v_threshold: float,
                                v_reset: Optional[float], detach_reset: bool = False, surrogate_function=None):
    return _run("plif", x_seq, v_init, r_tau, plan, 0.0, decay_input, v_threshold, v_reset, detach_reset,
                surrogate_function)


def _plan_for(kind: str, x_seq: torch.Tensor, storage_dtype, compute_dtype, backward_compute_dtype, spike_dtype,
              save_intermediates) -> HipNeuronExecutionPlan:
    return prepare_hip_neuron_execution_plan(neuron_type=kind, device=x_seq.device, storage_dtype=storage_dtype,
                                             forward_compute_dtype=compute_dtype,
                                             backward_compute_dtype=backward_compute_dtype, spike_dtype=spike_dtype,
                                             save_intermediates=save_intermediates)


def multistep_if_mp(x_seq: torch.Tensor, v_init: torch.Tensor, *, v_threshold: float, v_reset: Optional[float],
                    storage_dtype, compute_dtype="fp32", backward_compute_dtype="fp32",
                    spike_dtype: torch.dtype = torch.float32, save_intermediates: bool = True,
                    detach_reset: bool = False, surrogate_function=None):
    """Mixed-precision multi-step IF -> ``(s_seq, v_seq, h_seq | None)``."""
    plan = _plan_for("if", x_seq, storage_dtype, compute_dtype, backward_compute_dtype, spike_dtype, save_intermediates)
    return multistep_if_mp_with_plan(x_seq, v_init, plan, v_threshold=v_threshold, v_reset=v_reset,
                                     detach_reset=detach_reset, surrogate_function=surrogate_function)


def multistep_lif_mp(x_seq: torch.Tensor, v_init: torch.Tensor, *, decay_input: bool, tau: float, v_threshold: float,
                     v_reset: Optional[float], storage_dtype, compute_dtype="fp32", backward_compute_dtype="fp32",
                     spike_dtype: torch.dtype = torch.float32, save_intermediates: bool = True,
                     detach_reset: bool = False, surrogate_function=None):
    """Mixed-precision multi-step LIF -> ``(s_seq, v_seq, h_seq | None)``."""
    plan = _plan_for("lif", x_seq, storage_dtype, compute_dtype, backward_compute_dtype, spike_dtype, save_intermediates)
    return multistep_lif_mp_with_plan(x_seq, v_init, plan, decay_input=decay_input, tau=tau, v_threshold=v_threshold,
                                      v_reset=v_reset, detach_reset=detach_reset, surrogate_function=surrogate_function)


def multistep_plif_mp(x_seq: torch.Tensor, v_init: torch.Tensor, r_tau: torch.Tensor, *, decay_input: bool,
                      v_threshold: float, v_reset: Optional[float], storage_dtype, compute_dtype="fp32",
                      backward_compute_dtype="fp32", spike_dtype: torch.dtype = torch.float32,
                      save_intermediates: bool = True, detach_reset: bool = False, surrogate_function=None):
    """Mixed-precision multi-step parametric LIF (``r_tau`` = ``sigmoid(w)``, a 0-dim tensor on the device)
    -> ``(s_seq, v_seq, h_seq | None)``."""
    plan = _plan_for("plif", x_seq, storage_dtype, compute_dtype, backward_compute_dtype, spike_dtype, save_intermediates)
    return multistep_plif_mp_with_plan(x_seq, v_init, r_tau, plan, decay_input=decay_input, v_threshold=v_threshold,
                                       v_reset=v_reset, detach_reset=detach_reset, surrogate_function=surrogate_function)
