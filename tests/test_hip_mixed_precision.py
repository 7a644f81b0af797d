"""Mixed-precision IF / LIF / PLIF (``hip_kernel/neuron_mp_kernel.py``): 8-bit floating-point storage on its own
kernels, 16- and 32-bit storage routed to the ordinary ones.

Oracle: the reference's recipe for these operators (``test/activation_based/test_triton_neuron.py:212-247``, restated in
``oracle/neuron_oracle.py::multi_step_mixed_precision``): inputs rounded to the storage dtype by torch's CPU conversion,
fp32 arithmetic, stored values rounded.  Bars: spikes bit-exact, stored ``v_seq`` / ``h_seq`` equal byte for byte;
gradients within rtol 1e-5 of the closed-form BPTT (``oracle/bptt_oracle.py``, pinned against autograd elsewhere) run on
the stored ``h_seq`` the kernel itself reads.
"""

import numpy as np
import pytest
import torch

from oracle import bptt_oracle as bo
from oracle import neuron_oracle as no
from spikingjelly_amd.activation_based import surrogate
from spikingjelly_amd.activation_based.hip_kernel import library as L
from spikingjelly_amd.activation_based.hip_kernel import neuron_mp_kernel as M

from helpers import bits_equal, seeded_randn

F8 = [torch.float8_e4m3fn, torch.float8_e5m2]


# ---- host logic (no GPU) ----------------------------------------------------------------------------------------------

def test_dtype_names_follow_the_reference_rules():
    assert M.normalize_storage_dtype("torch.float8_e4m3fn") is torch.float8_e4m3fn
    assert M.normalize_storage_dtype("bf16") is torch.bfloat16 and M.normalize_storage_dtype(torch.float16) is torch.float16
    with pytest.raises(ValueError, match="ambiguous"):
        M.normalize_storage_dtype("fp8")
    with pytest.raises(ValueError, match="Unsupported"):
        M.normalize_storage_dtype(torch.float64)
    with pytest.raises(ValueError, match="string or torch.dtype"):
        M.normalize_storage_dtype(8)
    assert M.normalize_compute_dtype_name(torch.float8_e4m3fn) == "fp8" == M.normalize_compute_dtype_name(torch.float8_e5m2)
    assert M.normalize_compute_dtype_name("FP32") == "fp32" and M.normalize_compute_dtype_name(torch.bfloat16) == "bf16"
    assert M.is_fp8_dtype(torch.float8_e5m2) and not M.is_fp8_dtype(torch.float16)


def test_plan_validation():
    plan = M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda:0", storage_dtype="float8_e4m3fn",
                                               spike_dtype=torch.bfloat16)
    assert plan.storage_dtype is torch.float8_e4m3fn and plan.forward_compute_dtype_name == "fp32"
    assert plan.matches(neuron_type="lif", device=0, storage_dtype=torch.float8_e4m3fn, forward_compute_dtype="fp32",
                        spike_dtype=torch.bfloat16, save_intermediates=True)
    assert not plan.matches(neuron_type="if", device=0, storage_dtype=torch.float8_e4m3fn, forward_compute_dtype="fp32",
                            spike_dtype=torch.bfloat16, save_intermediates=True)
    assert not plan.matches(neuron_type="lif", device=0, storage_dtype="fp8", forward_compute_dtype="fp32",
                            spike_dtype=torch.bfloat16, save_intermediates=True)
    assert M.prepare_hip_neuron_execution_plan(neuron_type="if", device="cuda:0", storage_dtype="bf16",
                                               forward_compute_dtype="bf16").round_every_op
    with pytest.raises(ValueError, match="neuron_type"):
        M.prepare_hip_neuron_execution_plan(neuron_type="qif", device="cuda:0", storage_dtype="bf16")
    with pytest.raises(ValueError, match="requires an FP8 storage_dtype"):
        M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda:0", storage_dtype="bf16", forward_compute_dtype="fp8")
    with pytest.raises(ValueError, match="backward_compute_dtype='fp8'"):
        M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda:0", storage_dtype="bf16", backward_compute_dtype="fp8")
    with pytest.raises(ValueError, match="spike_dtype"):
        M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda:0", storage_dtype="bf16", spike_dtype=torch.int8)
    with pytest.raises(ValueError, match="save_intermediates"):
        M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda:0", storage_dtype="bf16", save_intermediates=1)
    with pytest.raises(RuntimeError, match="device"):
        M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cpu", storage_dtype="bf16")
    with pytest.raises(NotImplementedError, match="compute_dtype='fp8'"):
        M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda:0", storage_dtype="float8_e5m2", forward_compute_dtype="fp8")
    with pytest.raises(NotImplementedError, match="compute_dtype='bf16'"):
        M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda:0", storage_dtype="fp16", forward_compute_dtype="bf16")
    with pytest.raises(NotImplementedError, match="backward_compute_dtype='fp16'"):
        M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda:0", storage_dtype="fp16", backward_compute_dtype="fp16")


def test_cpu_tensors_are_refused():
    plan = M.prepare_hip_neuron_execution_plan(neuron_type="if", device="cuda:0", storage_dtype="float8_e5m2")
    with pytest.raises(RuntimeError, match="ROCm device"):
        M.multistep_if_mp_with_plan(torch.zeros(2, 4), torch.zeros(4), plan, v_threshold=1.0, v_reset=0.0)


# ---- GPU --------------------------------------------------------------------------------------------------------------

def _codes(t):
    return t.detach().cpu().contiguous().view(torch.uint8)


def _same_stored(got, want):
    """Byte for byte, except that any NaN code stands for any other (the formats have several; which one a conversion
    emits carries no information)."""
    a, b = got.detach().cpu().contiguous(), want.detach().cpu().contiguous()
    nan_a, nan_b = torch.isnan(a.float()), torch.isnan(b.float())
    return bool(torch.equal(nan_a, nan_b)) and bool(torch.equal(_codes(a)[~nan_a], _codes(b)[~nan_b]))


def _call(kind, x, v0, k, **kw):
    if kind == "if":
        return M.multistep_if_mp(x, v0, **kw)
    if kind == "lif":
        return M.multistep_lif_mp(x, v0, decay_input=kw.pop("decay_input"), tau=1.0 / k, **kw)
    return M.multistep_plif_mp(x, v0, torch.tensor(k, device=x.device), decay_input=kw.pop("decay_input"), **kw)


@pytest.mark.gpu
@pytest.mark.parametrize("storage", F8)
@pytest.mark.parametrize("kind,k,decay_input", [("if", 0.0, True), ("lif", 0.5, True), ("lif", 0.5, False), ("lif", 0.25, True),
                                                ("lif", 0.25, False), ("plif", 0.5744425, True), ("plif", 0.5744425, False)])
@pytest.mark.parametrize("v_reset", [0.0, -0.25, None])
@pytest.mark.parametrize("spike_dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_fp8_forward_equals_the_recipe(storage, kind, k, v_reset, decay_input, spike_dtype):
    T, N = 9, 1000  # not a multiple of 16: the operator pads
    x = seeded_randn((T, N), 41, 0.9, 1.0)
    v0 = seeded_randn((N,), 42, 0.0, 0.3)
    es, ev, eh = no.multi_step_mixed_precision(kind, x, v0, storage, k=k, decay_input=decay_input, v_reset=v_reset)
    kw = dict(v_threshold=1.0, v_reset=v_reset, storage_dtype=storage, spike_dtype=spike_dtype)
    if kind != "if":
        kw["decay_input"] = decay_input
    with torch.no_grad():
        s, v_seq, h_seq = _call(kind, x.cuda(), v0.cuda(), k, **kw)
    assert s.dtype == spike_dtype and v_seq.dtype == storage and h_seq.dtype == storage and s.shape == x.shape
    assert bits_equal(s.float().cpu(), es) and 0.01 < float(es.mean()) < 0.9
    assert _same_stored(v_seq, ev.to(storage)) and _same_stored(h_seq, eh.to(storage))


@pytest.mark.gpu
@pytest.mark.parametrize("storage", F8)
def test_fp8_codes_survive_the_kernel_and_the_input_cast_is_torchs(storage):
    """Every code of the format, decoded and stored again by the kernel, comes back unchanged (NaN included); and the
    operator's cast of its fp32 input (values of every binade, subnormals, halfway cases, the overflow rule: e4m3fn
    NaN, e5m2 infinity) gives the bytes of torch's CPU conversion."""
    every_code = torch.arange(256, dtype=torch.uint8).view(storage).float()
    finite = every_code[torch.isfinite(every_code)]
    ties = (finite[:-1] + finite[1:]) / 2
    top = float(finite.abs().max())
    wide = torch.cat([every_code, ties, ties * (1 + 2 ** -20), ties * (1 - 2 ** -20),
                      torch.tensor([top * 1.03, top * 1.04, top * 1.1, top * 4, 1e30, -1e30]),
                      seeded_randn((4096,), 43) * 3, seeded_randn((4096,), 44) * 2 ** -8, seeded_randn((2048,), 45) * 200])
    wide = wide[: wide.numel() // 16 * 16]
    x = torch.stack([wide * 0.0, wide])  # an IF neuron that never fires: h_1 = 0 + x_1
    x[0] = 0.0
    with torch.no_grad():
        s, v_seq, h_seq = M.multistep_if_mp(x.cuda(), torch.zeros_like(wide).cuda(), v_threshold=3e38, v_reset=None,
                                            storage_dtype=storage)
    want = (wide.to(storage).float() + 0.0).to(storage)  # the step's own h = 0 + x (-0 becomes +0)
    assert _same_stored(h_seq[1], want)
    assert _same_stored(x.cuda().to(storage), x.to(storage))


@pytest.mark.gpu
@pytest.mark.parametrize("storage", F8)
def test_fp8_kernel_rounds_fp32_values_like_torch(storage):
    """h = v + x with both operands on the storage grid is generally off the grid: the store rounds a genuine fp32 value."""
    N = 8192
    x = seeded_randn((3, N), 46, 0.0, 1.5)
    v0 = seeded_randn((N,), 47, 0.0, 1.5)
    es, ev, eh, raw = no.multi_step_mixed_precision("if", x, v0, storage, v_threshold=3e38, v_reset=None, return_raw_h=True)
    assert float((raw != eh).float().mean()) > 0.3  # most sums needed rounding
    with torch.no_grad():
        _, v_seq, h_seq = M.multistep_if_mp(x.cuda(), v0.cuda(), v_threshold=3e38, v_reset=None, storage_dtype=storage)
    assert _same_stored(h_seq, raw.to(storage)) and _same_stored(v_seq, ev.to(storage))


@pytest.mark.gpu
@pytest.mark.parametrize("storage", F8)
@pytest.mark.parametrize("tau", [2.0, 4.0, 8.0, 3.0])
def test_fp8_store_rounds_ties_subnormals_and_overflow_like_torch(storage, tau):
    """A LIF neuron from v = 0 stores round(x / tau): halving and quartering every code of the format lands on every
    halfway point between neighbours (also among the subnormals and below the smallest one), tau = 3 on values off any
    grid; doubling through a negative reset covers the overflow rule.  Expected bytes: torch's CPU conversion."""
    every_code = torch.arange(256, dtype=torch.uint8).view(storage).float()
    x = every_code[torch.isfinite(every_code)]
    x = torch.cat([x, x[:2]])[None]  # 254 or 248 finite codes, padded to a multiple of 16 by the operator anyway
    with torch.no_grad():
        _, _, h_seq = M.multistep_lif_mp(x.cuda(), torch.zeros_like(x[0]).cuda(), decay_input=True, tau=tau, v_threshold=3e38,
                                         v_reset=0.0, storage_dtype=storage)
    assert _same_stored(h_seq, (0.0 + x / tau).to(storage))  # the charge ends in v + ..., so -0 becomes +0
    # v = h = 2 x (IF from v0 = x): everything above half the largest finite value overflows
    with torch.no_grad():
        _, _, h_seq = M.multistep_if_mp(x.cuda(), x[0].cuda(), v_threshold=3e38, v_reset=None, storage_dtype=storage)
    want = (x + x).to(storage)
    assert _same_stored(h_seq, want)
    assert bool(torch.isnan(want.float()).any() or torch.isinf(want.float()).any())


SG = {"sigmoid": (surrogate.Sigmoid, 4.0), "atan": (surrogate.ATan, 2.0), "erf": (surrogate.Erf, 2.0)}


@pytest.mark.gpu
@pytest.mark.parametrize("storage", F8)
@pytest.mark.parametrize("kind,k,decay_input", [("if", 0.0, True), ("lif", 0.5, True), ("lif", 0.5, False),
                                                ("plif", 0.5744425, True), ("plif", 0.5744425, False)])
@pytest.mark.parametrize("v_reset,detach", [(0.0, False), (-0.25, True), (None, False)])
@pytest.mark.parametrize("sg_name,spike_dtype", [("sigmoid", torch.float32), ("atan", torch.bfloat16), ("erf", torch.float16)])
def test_fp8_backward_equals_the_closed_form_on_the_stored_h(storage, kind, k, v_reset, detach, decay_input, sg_name, spike_dtype):
    T, N = 7, 520
    x = seeded_randn((T, N), 51, 0.4, 0.7).cuda().requires_grad_()
    v0 = seeded_randn((N,), 52, 0.0, 0.3).cuda().requires_grad_()
    kt = torch.tensor(k, device="cuda", requires_grad=(kind == "plif"))
    cls, alpha = SG[sg_name]
    kw = dict(v_threshold=1.0, v_reset=v_reset, storage_dtype=storage, spike_dtype=spike_dtype, detach_reset=detach,
              surrogate_function=cls(alpha))
    if kind == "if":
        s, v_seq, h_seq = M.multistep_if_mp(x, v0, **kw)
    elif kind == "lif":
        s, v_seq, h_seq = M.multistep_lif_mp(x, v0, decay_input=decay_input, tau=1.0 / k, **kw)
    else:
        s, v_seq, h_seq = M.multistep_plif_mp(x, v0, kt, decay_input=decay_input, **kw)
    gs = seeded_randn((T, N), 53).to(spike_dtype)
    gv = seeded_randn((T, N), 54, 0.0, 0.2).to(storage)
    torch.autograd.backward([s, v_seq], [gs.cuda(), gv.cuda()])
    assert x.grad.dtype == torch.float32 and v0.grad.shape == v0.shape
    # the closed form on what the kernel reads: stored h, spikes recomputed from it, the rounded upstream gradients
    h = h_seq.detach().float().cpu().double().numpy()
    vq = v0.detach().to(storage).float().cpu().double().numpy()
    vr = 0.0 if v_reset is None else v_reset
    spikes = (h >= 1.0).astype(np.float64)
    v_after = (h - spikes) if v_reset is None else (spikes * vr + (1.0 - spikes) * h)
    v_prev = np.concatenate([vq[None], v_after[:-1]])
    x_eff = None
    if kind == "plif" and decay_input:
        # the kernel uses (h_t - v_{t-1}) / k for dh/dk; the closed form's x_t - (v_{t-1} - vr) equals it
        x_eff = (h - v_prev) / k + (v_prev - vr)
    sgp = lambda z: no.surrogate_grad(sg_name, torch.from_numpy(z), alpha).numpy()
    want_x, want_v0, want_k = bo.bptt(kind, h, spikes, sgp, gs.float().double().numpy(), gv.float().double().numpy(), None,
                                      k, decay_input, 1.0, v_reset, detach, v_prev_seq=v_prev, x_seq=x_eff)
    np.testing.assert_allclose(x.grad.cpu().double().numpy(), want_x, rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(v0.grad.cpu().double().numpy(), want_v0, rtol=2e-5, atol=2e-6)
    if kind == "plif":
        np.testing.assert_allclose(float(kt.grad), want_k, rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("storage", F8)
@pytest.mark.parametrize("neuron_id,k", [(0, None), (1, None), (2, 0.5744425)])
@pytest.mark.parametrize("N", [512, 520, 37])
def test_fp8_gradients_written_in_the_storage_dtype_are_the_rounded_fp32_ones(storage, neuron_id, k, N):
    """What the reference does (it allocates grad_x_seq / grad_v_init in the dtypes of x_seq / v_init,
    triton_kernel/neuron_kernel/lif.py:1115-1118): the kernel rounds its fp32 value once, so the result is the cast of
    the fp32 result, at 5 instead of 8 bytes per neuron-step."""
    T = 6
    h = seeded_randn((T, N), 61, 0.6, 0.7).cuda().to(storage)
    v0 = seeded_randn((N,), 62, 0.0, 0.3).cuda().to(storage)
    gs = seeded_randn((T, N), 63).cuda().to(torch.bfloat16)
    gv = seeded_randn((T, N), 64, 0.0, 0.2).cuda().to(storage)
    kt = None if k is None else torch.tensor(k, device="cuda")
    neuron = (L.NEURON_IF, L.NEURON_LIF, L.NEURON_PLIF)[neuron_id]
    scalars = (neuron, 2.0, True, 1.0, 0.0, False, False, 1, 2.0)
    wide = M.hip_multistep_mp_backward(gs, gv, h, v0, kt, *scalars, torch.bfloat16, False)
    narrow = M.hip_multistep_mp_backward(gs, gv, h, v0, kt, *scalars, torch.bfloat16, True)
    assert wide[0].dtype == torch.float32 and narrow[0].dtype == storage and narrow[1].dtype == storage
    assert narrow[0].shape == (T, N) and narrow[1].shape == (N,)
    assert _same_stored(narrow[0], wide[0].to(storage)) and _same_stored(narrow[1], wide[1].to(storage))
    assert bits_equal(narrow[2], wide[2]) and float(wide[0].abs().sum()) > 0


@pytest.mark.gpu
@pytest.mark.parametrize("storage", F8)
def test_fp8_inputs_get_fp8_gradients_through_autograd(storage):
    T, N = 5, 256
    x32 = seeded_randn((T, N), 71, 0.4, 0.7).cuda()
    v32 = seeded_randn((N,), 72, 0.0, 0.3).cuda()
    gs = seeded_randn((T, N), 73).cuda()
    kw = dict(decay_input=True, tau=2.0, v_threshold=1.0, v_reset=0.0, storage_dtype=storage, spike_dtype=torch.float32,
              surrogate_function=surrogate.ATan(2.0))
    x8, v8 = x32.to(storage).requires_grad_(), v32.to(storage).requires_grad_()
    s8, _, _ = M.multistep_lif_mp(x8, v8, **kw)
    s8.backward(gs)
    # the same values fed as fp32 tensors take the fp32 route; its gradients, cast, are the fp8 route's
    xw, vw = x8.detach().float().requires_grad_(), v8.detach().float().requires_grad_()
    sw, _, _ = M.multistep_lif_mp(xw, vw, **kw)
    sw.backward(gs)
    assert bits_equal(s8.detach(), sw.detach())
    assert x8.grad.dtype == storage and v8.grad.dtype == storage
    assert _same_stored(x8.grad, xw.grad.to(storage)) and _same_stored(v8.grad, vw.grad.to(storage))


@pytest.mark.gpu
@pytest.mark.parametrize("storage,compute", [(torch.bfloat16, "fp32"), (torch.float16, "fp32"), (torch.float32, "fp32"),
                                             (torch.bfloat16, "bf16"), (torch.float16, "fp16")])
@pytest.mark.parametrize("kind,k", [("if", 0.0), ("lif", 0.5), ("plif", 0.5744425)])
def test_wider_storage_runs_the_ordinary_kernels(storage, compute, kind, k):
    T, N = 8, 777
    x, v0 = seeded_randn((T, N), 61, 0.4, 0.7), seeded_randn((N,), 62, 0.0, 0.3)
    kw = dict(v_threshold=1.0, v_reset=0.0, storage_dtype=storage, compute_dtype=compute, spike_dtype=torch.float32)
    if kind != "if":
        kw["decay_input"] = True
    with torch.no_grad():
        s, v_seq, h_seq = _call(kind, x.cuda(), v0.cuda(), k, **kw)
    assert s.dtype == torch.float32 and v_seq.dtype == storage and h_seq.dtype == storage
    if compute == "fp32":
        es, ev, eh = no.multi_step_mixed_precision(kind, x, v0, storage, k=k, v_reset=0.0)
        assert bits_equal(s.cpu(), es) and bits_equal(v_seq.float().cpu(), ev) and bits_equal(h_seq.float().cpu(), eh)
    else:  # every op rounded: the torch backend on half tensors
        tau_or_w = None if kind == "if" else (1.0 / k if kind == "lif" else torch.tensor(k).logit())
        if kind != "plif":  # (the oracle's PLIF recomputes k from w; a last-bit difference in k is not the subject here)
            es, ev, eh = no.multi_step(kind, x.to(storage), v0.to(storage), tau_or_w, True, 1.0, 0.0)
            assert bits_equal(s.cpu(), es.float()) and bits_equal(v_seq.cpu(), ev)
    # and training through them
    xg = x.cuda().requires_grad_()
    s, v_seq, h_seq = _call(kind, xg, v0.cuda(), k, **dict(kw, surrogate_function=surrogate.ATan()))
    s.sum().backward()
    assert xg.grad is not None and xg.grad.dtype == torch.float32 and bool(torch.isfinite(xg.grad).all())


@pytest.mark.gpu
def test_save_intermediates_false_returns_no_h_and_plans_are_reusable():
    plan = M.prepare_hip_neuron_execution_plan(neuron_type="lif", device="cuda", storage_dtype=torch.float8_e4m3fn,
                                               spike_dtype=torch.bfloat16, save_intermediates=False)
    x, v0 = seeded_randn((4, 64), 71, 0.4, 0.7).cuda(), torch.zeros(64, device="cuda")
    for _ in range(2):
        with torch.no_grad():
            s, v_seq, h_seq = M.multistep_lif_mp_with_plan(x, v0, plan, decay_input=True, tau=2.0, v_threshold=1.0, v_reset=0.0)
        assert h_seq is None and s.dtype == torch.bfloat16 and v_seq.dtype == torch.float8_e4m3fn
    with pytest.raises(ValueError, match="requires a IF plan|requires a"):
        M.multistep_if_mp_with_plan(x, v0, plan, v_threshold=1.0, v_reset=0.0)
    with pytest.raises(RuntimeError, match="v_init shape"):
        M.multistep_lif_mp_with_plan(x, v0[:32], plan, decay_input=True, tau=2.0, v_threshold=1.0, v_reset=0.0)


@pytest.mark.gpu
def test_mp_operators_pass_opcheck():
    x = seeded_randn((4, 64), 81, 0.4, 0.7).cuda().requires_grad_()
    v0 = torch.zeros(64, device="cuda", requires_grad=True)
    args = (x, v0, None, 1, 2.0, True, 1.0, 0.0, False, False, 1, 2.0, torch.float8_e4m3fn, torch.bfloat16, True)
    # (the schema test clones and compares outputs with arithmetic torch does not have for 8-bit floats)
    torch.library.opcheck(M.hip_multistep_mp_forward, args, test_utils=("test_faketensor", "test_autograd_registration"))
