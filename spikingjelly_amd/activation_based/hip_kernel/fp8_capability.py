"""What the hip backend can do with 8-bit floating-point storage on a device, found by running it.

Counterpart of the reference's ``triton_kernel/fp8_capability.py`` (probes :130-267, public functions :318-424): the same
questions (is ``float8_e4m3fn`` / ``float8_e5m2`` storage usable for a neuron's forward / backward with a given compute
dtype on this device?), the same answers' shape (``{"available": bool, "reason": str | None}``, and a report over every
storage and compute dtype), asked of ``libsjhip.so`` instead of a Triton compile.  A probe runs the real mixed-precision
operators on eight values and checks what comes back, so a missing library, a device the library was not built for or
a broken conversion all show up here, with the reason, instead of inside a training step.  Results are cached per
(dtype, device, compute dtype, torch version).

Only fp32 arithmetic is built: the other compute dtypes of the reference's experimental operators are reported
unavailable with that reason (``prepare_hip_neuron_execution_plan`` refuses them likewise).
"""

from __future__ import annotations

import copy
import functools
import threading
import traceback
from typing import Any

import torch

from ...logger import logger
from . import library as L
from .neuron_mp_kernel import is_fp8_dtype, normalize_compute_dtype_name, normalize_storage_dtype

__all__ = [
    "supports_hip_fp8_e4m3fn",
    "supports_hip_fp8_e5m2",
    "supports_hip_fp8_neuron_forward",
    "supports_hip_fp8_neuron_backward",
    "hip_fp8_neuron_capability",
    "hip_fp8_neuron_backward_capability",
    "hip_fp8_neuron_capability_report",
]

_PROBE_VALUES = [0.0, 0.25, -0.5, 1.0, 2.0, -2.0, 0.75, -0.75]
_per_thread = threading.local()


def probing() -> bool:
    """True while a probe runs on the calling thread (plan preparation then skips its own capability check)."""
    return getattr(_per_thread, "probing", False)


def _fp8_dtype_candidates() -> dict[str, Any]:
    return {"torch.float8_e4m3fn": getattr(torch, "float8_e4m3fn", None),
            "torch.float8_e5m2": getattr(torch, "float8_e5m2", None)}


def _answer(available: bool, reason: str | None = None) -> dict[str, Any]:
    return {"available": available, "reason": reason}


def _reason_of(e: Exception) -> str:
    return traceback.format_exception_only(type(e), e)[-1].strip()


def _normalize_fp8_dtype(dtype) -> torch.dtype:
    try:
        normalized = normalize_storage_dtype(dtype)
    except ValueError as e:
        raise ValueError(f"Unsupported hip FP8 dtype: {dtype!r}.") from e
    if not is_fp8_dtype(normalized):
        raise ValueError(f"Unsupported hip FP8 dtype: {normalized}.")
    return normalized


def _library_loads() -> bool:
    try:
        L.load()
    except Exception:
        return False
    return True


def _normalize_device(device) -> torch.device:
    device = torch.device(device)
    if device.type == "cuda" and device.index is None and torch.cuda.is_available():
        device = torch.device("cuda", torch.cuda.current_device())
    return device


@functools.lru_cache(maxsize=None)
def _probe_cached(dtype_name: str, device_str: str, compute_dtype_name: str, backward: bool, torch_version: str):
    del torch_version  # a cache key only: a new torch may bring other conversions
    what = "backward" if backward else "forward"
    try:
        dtype = _normalize_fp8_dtype(dtype_name)
        compute = normalize_compute_dtype_name(compute_dtype_name)
    except ValueError as e:
        return _answer(False, str(e))
    if compute != "fp32":
        return _answer(False, f"the hip neuron kernels compute in fp32; compute dtype {compute!r} is not built")
    if not torch.cuda.is_available():
        return _answer(False, "no ROCm device is available")
    device = _normalize_device(device_str)
    if device.type != "cuda":
        return _answer(False, f"hip FP8 neuron {what} requires a ROCm device")
    try:
        L.load()
    except Exception as e:
        return _answer(False, _reason_of(e))
    _per_thread.probing = True
    try:
        from . import neuron_mp_kernel as M
        from .. import surrogate

        x32 = torch.tensor([_PROBE_VALUES, _PROBE_VALUES[::-1]], device=device, dtype=torch.float32)
        x = x32.to(dtype).requires_grad_(backward)
        v0 = torch.zeros(x.shape[1], device=device, dtype=dtype)
        s, v_seq, _ = M.multistep_lif_mp(x, v0, decay_input=True, tau=2.0, v_threshold=1.0, v_reset=0.0,
                                        storage_dtype=dtype, spike_dtype=torch.float32,
                                        surrogate_function=surrogate.ATan(2.0))
        # the recurrence on these values in fp32, stored values rounded like the operator's
        v, want_s, want_v = torch.zeros_like(x32[0]), [], []
        for t in range(x32.shape[0]):
            h = v + (x32[t] - v) / 2.0
            spike = (h >= 1.0).float()
            v = ((1.0 - spike) * h).to(dtype).float()
            want_s.append(spike)
            want_v.append(v)
        if not torch.equal(s.detach(), torch.stack(want_s)) or not torch.equal(v_seq.detach().float(), torch.stack(want_v)):
            return _answer(False, "probe produced values that differ from the fp32 recurrence on rounded storage")
        if backward:
            s.sum().backward()
            grad = x.grad
            if grad is None or grad.dtype != dtype or not bool(torch.isfinite(grad.float()).all()):
                return _answer(False, "probe produced no finite gradient in the storage dtype")
        torch.cuda.synchronize(device)
    except Exception as e:
        return _answer(False, _reason_of(e))
    finally:
        _per_thread.probing = False
    return _answer(True)


def _probe(dtype, device, compute_dtype="fp32", backward: bool = False) -> dict[str, Any]:
    try:
        dtype_name = str(_normalize_fp8_dtype(dtype))
    except ValueError as e:
        return _answer(False, str(e))
    return dict(_probe_cached(dtype_name, str(_normalize_device(device)), str(compute_dtype), backward, torch.__version__))


def supports_hip_fp8_e4m3fn(device) -> bool:
    dtype = getattr(torch, "float8_e4m3fn", None)
    return False if dtype is None else bool(_probe(dtype, device)["available"])


def supports_hip_fp8_e5m2(device) -> bool:
    dtype = getattr(torch, "float8_e5m2", None)
    return False if dtype is None else bool(_probe(dtype, device)["available"])


def supports_hip_fp8_neuron_forward(dtype, device, compute_dtype="fp32") -> bool:
    return bool(_probe(dtype, device, compute_dtype)["available"])


def supports_hip_fp8_neuron_backward(dtype, device, compute_dtype="fp32") -> bool:
    return bool(_probe(dtype, device, compute_dtype, backward=True)["available"])


def hip_fp8_neuron_capability(dtype, device, compute_dtype="fp32") -> dict[str, Any]:
    return _probe(dtype, device, compute_dtype)


def hip_fp8_neuron_backward_capability(dtype, device, compute_dtype="fp32") -> dict[str, Any]:
    return _probe(dtype, device, compute_dtype, backward=True)


def hip_fp8_neuron_capability_report(device) -> dict[str, Any]:
    """Forward / backward availability, with reasons, of every FP8 storage dtype under every compute dtype on ``device``.

    ``dtypes`` holds the fp32-compute results (the reference's compatibility field), ``compute_dtypes`` all of them.
    """
    device = _normalize_device(device)
    report: dict[str, Any] = {
        "device": str(device),
        "device_type": device.type,
        "cuda_available": torch.cuda.is_available(),
        "hip_library_available": _library_loads(),
        "torch_version": torch.__version__,
        "hip_version": getattr(torch.version, "hip", None),
        "device_name": None,
        "dtypes": {},
        "compute_dtypes": {},
    }
    if device.type == "cuda" and torch.cuda.is_available():
        report["device_name"] = torch.cuda.get_device_name(device)
    for compute_dtype in ("fp32", "fp16", "bf16", "fp8"):
        per_dtype = {}
        for name, dtype in _fp8_dtype_candidates().items():
            if dtype is None:
                forward = backward = _answer(False, f"{name} is unavailable in this PyTorch build")
            else:
                forward = _probe(dtype, device, compute_dtype)
                backward = _probe(dtype, device, compute_dtype, backward=True)
            per_dtype[name] = {"forward": forward, "backward": backward}
        report["compute_dtypes"][compute_dtype] = per_dtype
    report["dtypes"] = copy.deepcopy(report["compute_dtypes"]["fp32"])
    logger.info("hip_fp8_capability_summary device=%s library=%s rocm=%s", device, report["hip_library_available"],
                report["cuda_available"])
    return report
