"""The FP8 capability probes of the hip backend (counterpart of the reference's triton_kernel/fp8_capability.py,
public functions :318-424): answers have the reference's shape, and on a GPU they come from running the kernels."""

import pytest
import torch

from spikingjelly_amd.activation_based.hip_kernel import fp8_capability as C

F8 = [torch.float8_e4m3fn, torch.float8_e5m2]


def test_answers_without_a_gpu_give_the_reason():
    for dtype in F8:
        for ask in (C.hip_fp8_neuron_capability, C.hip_fp8_neuron_backward_capability):
            got = ask(dtype, "cpu")
            assert got["available"] is False and "ROCm device" in got["reason"]
    assert C.supports_hip_fp8_neuron_forward(torch.float8_e5m2, "cpu") is False
    assert C.supports_hip_fp8_neuron_backward("float8_e4m3fn", "cpu") is False


def test_what_is_not_an_fp8_dtype_is_refused_with_a_reason():
    for bad in (torch.float16, "fp8", "int8", 3):
        got = C.hip_fp8_neuron_capability(bad, "cpu")
        assert got["available"] is False and "Unsupported hip FP8 dtype" in got["reason"]
    got = C.hip_fp8_neuron_capability(torch.float8_e4m3fn, "cpu", compute_dtype="int4")
    assert got["available"] is False and got["reason"]


def test_compute_dtypes_that_are_not_built_say_so():
    for compute in ("fp16", "bf16", "fp8", torch.bfloat16):
        got = C.hip_fp8_neuron_capability(torch.float8_e4m3fn, "cpu", compute_dtype=compute)
        assert got["available"] is False and "compute in fp32" in got["reason"]


def test_report_has_the_reference_layout():
    report = C.hip_fp8_neuron_capability_report("cpu")
    assert report["device_type"] == "cpu" and set(report["compute_dtypes"]) == {"fp32", "fp16", "bf16", "fp8"}
    for per_dtype in report["compute_dtypes"].values():
        assert set(per_dtype) == {"torch.float8_e4m3fn", "torch.float8_e5m2"}
        for passes in per_dtype.values():
            assert set(passes) == {"forward", "backward"}
            assert all(set(a) == {"available", "reason"} for a in passes.values())
    assert report["dtypes"] == report["compute_dtypes"]["fp32"]
    report["dtypes"]["torch.float8_e5m2"]["forward"]["reason"] = "edited"  # a copy, not a view of the cache
    assert C.hip_fp8_neuron_capability(torch.float8_e5m2, "cpu")["reason"] != "edited"


@pytest.mark.gpu
def test_both_storage_dtypes_run_forward_and_backward_on_the_gpu():
    assert C.supports_hip_fp8_e4m3fn("cuda") and C.supports_hip_fp8_e5m2("cuda:0")
    for dtype in F8:
        assert C.hip_fp8_neuron_capability(dtype, "cuda") == {"available": True, "reason": None}
        assert C.hip_fp8_neuron_backward_capability(dtype, "cuda") == {"available": True, "reason": None}
        assert not C.supports_hip_fp8_neuron_forward(dtype, "cuda", compute_dtype="bf16")
    report = C.hip_fp8_neuron_capability_report("cuda")
    assert report["hip_library_available"] and report["device_name"]
    assert all(p["available"] for d in report["dtypes"].values() for p in d.values())
    assert not any(p["available"] for d in report["compute_dtypes"]["fp8"].values() for p in d.values())


def test_plan_preparation_refuses_what_the_probe_refuses(monkeypatch):
    """The reference checks the capability when a plan is prepared (triton_kernel/neuron_kernel/utils.py:99-152)."""
    from spikingjelly_amd.activation_based.hip_kernel import neuron_mp_kernel as M

    monkeypatch.setattr(C, "hip_fp8_neuron_capability", lambda *a, **k: {"available": False, "reason": "made up"})
    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: False)
    with pytest.raises(RuntimeError, match="hip FP8 LIF forward is unavailable for torch.float8_e5m2 .*made up"):
        M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda:0", storage_dtype=torch.float8_e5m2)
    # 16-bit storage asks nothing
    plan = M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda:0", storage_dtype=torch.bfloat16)
    assert plan.storage_dtype == torch.bfloat16
