"""Parity of the HIP kernels (through the C ABI of libsjhip.so) with the CPU oracle.

Bars: spikes / h / v bit-exact in fp32 and in "round every op" 16-bit mode; stored values exact after
rounding in fp32-state 16-bit mode; gradients within rtol 1e-5 (fp32) / 1e-2 (16-bit) of autograd
through the oracle.
"""

import math

import numpy as np
import pytest
import torch

from oracle import neuron_oracle as no

from helpers import bits_equal, load_dyadic, seeded_randn

pytestmark = pytest.mark.gpu

GRAD_RTOL, GRAD_ATOL = 1e-5, 1e-6     # fp32 gradients
HALF_RTOL = 1e-2                      # fp16 / bf16 gradients


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    from spikingjelly_amd.activation_based.hip_kernel import library, neuron_kernel

    library.load()
    return neuron_kernel


def _flags(fp32_state=False, reciprocal=False, atomic=False):
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    return (L.FLAG_FP32_STATE if fp32_state else 0) | (L.FLAG_RECIPROCAL_TAU if reciprocal else 0) | \
           (L.FLAG_ATOMIC_REDUCE if atomic else 0)


def hip_forward(K, kind, x, v0, tau_or_k, decay_input, vth, v_reset, store_v_seq=True, flags=0, training=True,
                recompute=False):
    """Calls the forward operator; returns CPU tensors (s, v_seq|None, v_last, h|None)."""
    soft = v_reset is None
    vr = 0.0 if soft else v_reset
    xd, vd = x.cuda(), v0.cuda()
    if kind == "if":
        out = (K.hip_multistep_if_forward(xd, vd, vth, vr, soft, False, 1, 2.0, store_v_seq, flags, recompute) if training
               else K.hip_multistep_if_inference(xd, vd, vth, vr, soft, store_v_seq, flags))
    elif kind == "lif":
        out = (K.hip_multistep_lif_forward(xd, vd, vth, vr, soft, False, tau_or_k, decay_input, 1, 2.0, store_v_seq, flags,
                                           recompute)
               if training else K.hip_multistep_lif_inference(xd, vd, vth, vr, soft, tau_or_k, decay_input, store_v_seq, flags))
    else:
        kd = torch.as_tensor(tau_or_k, dtype=torch.float32).cuda()
        out = (K.hip_multistep_plif_forward(xd, vd, kd, vth, vr, soft, False, decay_input, 1, 2.0, store_v_seq, flags,
                                            recompute)
               if training else K.hip_multistep_plif_inference(xd, vd, kd, vth, vr, soft, decay_input, store_v_seq, flags))
    torch.cuda.synchronize()
    s, v_seq, v_last = out[0].cpu(), (out[1].cpu() if store_v_seq else None), out[2].cpu()
    h = out[3].cpu() if training and not recompute else None
    if training and recompute:
        assert out[3].numel() == 0  # no h_seq is materialised on the replay path
    return s, v_seq, v_last, h


# ------------------------------------------------------------------------------------------------
# forward, fp32
# ------------------------------------------------------------------------------------------------
def test_dyadic_golden_vectors(K):
    doc = load_dyadic()
    for c in doc["cases"]:
        x = torch.tensor(doc["x"], dtype=torch.float32) * c["scale"]
        v0 = torch.tensor(doc["v_init"], dtype=torch.float32)
        p = {"if": 0.0, "lif": 1.0 / c["k"], "plif": c["k"]}[c["kind"]]
        for dtype, fl in ((torch.float32, 0), (torch.float16, 0), (torch.bfloat16, 0),
                          (torch.float16, _flags(fp32_state=True)), (torch.bfloat16, _flags(fp32_state=True))):
            s, v, vl, h = hip_forward(K, c["kind"], x.to(dtype), v0.to(dtype), p, c["decay_input"], c["v_threshold"],
                                      c["v_reset"], flags=fl)
            assert torch.equal(s.float(), torch.tensor(c["spike"])), (c["kind"], dtype)
            assert torch.equal(h.float(), torch.tensor(c["h"]))
            assert torch.equal(v.float(), torch.tensor(c["v"]))
            assert torch.equal(vl.float(), torch.tensor(c["v"])[-1])


FWD_GRID = [(kind, vr, di, tau)
            for kind in ("if", "lif", "plif")
            for vr in (0.0, -0.2, None)
            for di in ((True,) if kind == "if" else (True, False))
            for tau in ((2.0,) if kind == "if" else (2.0, 3.0, 10.0))]


@pytest.mark.parametrize("kind,v_reset,decay_input,tau", FWD_GRID)
@pytest.mark.parametrize("T,N", [(16, 8192), (7, 111), (65, 260), (1, 4), (4, 40)])
def test_forward_bit_exact_fp32(K, kind, v_reset, decay_input, tau, T, N):
    x = seeded_randn((T, N), 100 + T, 0.4, 1.0)
    v0 = seeded_randn((N,), 200 + N, 0.0, 0.3)
    vth = 0.8
    if kind == "plif":
        w = torch.tensor(-math.log(tau - 1.0))
        k = float(w.sigmoid())
        es, ev, eh = no.multi_step("plif", x, v0, w, decay_input, vth, v_reset)
        p = k
    else:
        es, ev, eh = no.multi_step(kind, x, v0, tau, decay_input, vth, v_reset)
        p = tau
    s, v, vl, h = hip_forward(K, kind, x, v0, p, decay_input, vth, v_reset)
    assert bits_equal(s, es)
    assert bits_equal(h, eh)
    assert bits_equal(v, ev)
    assert bits_equal(vl, ev[-1])
    # inference op (no h_seq) and last-state-only output give the same spikes and final state
    s2, v2, vl2, _ = hip_forward(K, kind, x, v0, p, decay_input, vth, v_reset, store_v_seq=False, training=False)
    assert v2 is None and bits_equal(s2, es) and bits_equal(vl2, ev[-1])


def test_forward_special_values(K):
    """Signed zeros, infinities, NaN and subnormals go through the arithmetic form of the reset."""
    row = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 1e-42, -1e-42, 3.0e38,
                        1.0, 0.99999994, 1.0000001, -1.0, 2.0, 1e-30, 5e-39, -5e-39], dtype=torch.float32)
    x = torch.stack([row, row.flip(0), row * 0.5, -row])
    v0 = torch.zeros(16)
    for kind, p in (("if", 0.0), ("lif", 2.0), ("lif", 3.0), ("plif", 0.25)):
        for v_reset in (0.0, -0.2, None):
            for di in (True, False):
                if kind == "plif":
                    w = torch.tensor(math.log(p / (1 - p)))
                    kf = float(w.sigmoid())
                    e = no.multi_step("plif", x, v0, w, di, 1.0, v_reset)
                    a = hip_forward(K, kind, x, v0, kf, di, 1.0, v_reset)
                else:
                    e = no.multi_step(kind, x, v0, p, di, 1.0, v_reset)
                    a = hip_forward(K, kind, x, v0, p, di, 1.0, v_reset)
                assert bits_equal(a[0], e[0]), (kind, v_reset, di)
                assert bits_equal(a[3], e[2]), (kind, v_reset, di)
                assert bits_equal(a[1], e[1]), (kind, v_reset, di)


def test_reciprocal_tau_flag_matches_multiplication(K):
    x = seeded_randn((8, 4096), 9, 0.4, 1.0)
    v0 = torch.zeros(4096)
    k = torch.tensor(float(np.float32(1.0 / 3.0)))
    e = no.multi_step("plif_k", x, v0, k, True, 1.0, 0.0)
    a = hip_forward(K, "lif", x, v0, 3.0, True, 1.0, 0.0, flags=_flags(reciprocal=True))
    assert bits_equal(a[0], e[0]) and bits_equal(a[3], e[2])


# ------------------------------------------------------------------------------------------------
# forward, 16-bit storage
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kind,v_reset,decay_input,tau", FWD_GRID)
@pytest.mark.parametrize("T,N", [(8, 4096), (5, 111)])
def test_forward_half_rounds_like_torch_backend(K, dtype, kind, v_reset, decay_input, tau, T, N):
    x = seeded_randn((T, N), 300 + T, 0.4, 1.0).to(dtype)
    v0 = seeded_randn((N,), 400 + N, 0.0, 0.3).to(dtype)
    vth = 0.7
    if kind == "plif":
        w = torch.tensor(-math.log(tau - 1.0))
        es, ev, eh = no.multi_step("plif", x, v0, w, decay_input, vth, v_reset)
        p = float(w.sigmoid())
    else:
        es, ev, eh = no.multi_step(kind, x, v0, tau, decay_input, vth, v_reset)
        p = tau
    assert es.dtype == dtype
    s, v, vl, h = hip_forward(K, kind, x, v0, p, decay_input, vth, v_reset)
    assert bits_equal(s, es)
    assert bits_equal(h, eh)
    assert bits_equal(v, ev)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kind,decay_input", [("if", True), ("lif", True), ("lif", False), ("plif", True), ("plif", False)])
@pytest.mark.parametrize("v_reset", [0.0, -0.2, None])
def test_forward_half_storage_fp32_state(K, dtype, kind, v_reset, decay_input):
    T, N, k = 8, 4096, 0.5
    x = seeded_randn((T, N), 500, 0.3, 1.0).to(dtype)
    v0 = seeded_randn((N,), 501, 0.0, 0.3).to(dtype)
    es, ev, eh = no.multi_step_mixed_precision(kind, x.float(), v0.float(), dtype, k, decay_input, 1.0, v_reset)
    p = {"if": 0.0, "lif": 1.0 / k, "plif": k}[kind]
    s, v, vl, h = hip_forward(K, kind, x, v0, p, decay_input, 1.0, v_reset, flags=_flags(fp32_state=True))
    assert torch.equal(s.float(), es)
    assert torch.equal(h.float(), eh)
    assert torch.equal(v.float(), ev)


# ------------------------------------------------------------------------------------------------
# backward
# ------------------------------------------------------------------------------------------------
def hip_backward(K, kind, gs, gv, gl, h, v0, tau_or_k, decay_input, vth, v_reset, detach, sg_id, alpha, flags=0,
                 x=None):
    """h given -> the kernel reads h_seq; x given (h None) -> the kernel replays the forward from x, v0."""
    soft = v_reset is None
    vr = 0.0 if soft else v_reset
    d = lambda t: None if t is None else t.cuda()
    hx = (d(h), None, None) if x is None else (None, d(x), d(v0))
    if kind == "if":
        out = K.hip_multistep_if_backward(d(gs), d(gv), d(gl), *hx, vth, vr, soft, detach, sg_id, alpha, flags)
    elif kind == "lif":
        out = K.hip_multistep_lif_backward(d(gs), d(gv), d(gl), *hx, vth, vr, soft, detach, tau_or_k, decay_input,
                                           sg_id, alpha, flags)
    else:
        kd = torch.as_tensor(tau_or_k, dtype=torch.float32).cuda()
        out = K.hip_multistep_plif_backward(d(gs), d(gv), d(gl), hx[0], hx[1], d(v0), kd, vth, vr, soft, detach,
                                            decay_input, sg_id, alpha, flags)
    torch.cuda.synchronize()
    return tuple(o.cpu() for o in out)


BWD_GRID = [(kind, sg, di, vr, det)
            for kind in ("if", "lif", "plif")
            for sg in ("atan", "sigmoid")
            for di in ((True,) if kind == "if" else (True, False))
            for vr in (0.0, -0.2, None)
            for det in (False, True)]


@pytest.mark.parametrize("kind,sg,decay_input,v_reset,detach", BWD_GRID)
@pytest.mark.parametrize("T,N,path", [(16, 4096, "h_seq"), (16, 4096, "replay"), (7, 111, "h_seq")])  # replay: N % 4 == 0
def test_backward_matches_autograd_fp32(K, kind, sg, decay_input, v_reset, detach, T, N, path):
    tau, vth = 3.0, 0.8
    alpha = no.SG_DEFAULT_ALPHA[sg]
    x = seeded_randn((T, N), 600 + T, 0.4, 1.0)
    v0 = seeded_randn((N,), 601, 0.0, 0.3)
    gs, gv, gl = seeded_randn((T, N), 602), seeded_randn((T, N), 603, 0, 0.1), seeded_randn((N,), 604, 0, 0.1)
    if kind == "plif":
        kt = torch.tensor(float(np.float32(1.0 / tau)))
        ref = no.forward_backward("plif_k", x, v0, gs, gv, gl, kt, decay_input, vth, v_reset, sg, alpha, detach)
        p = float(kt)
    else:
        ref = no.forward_backward(kind, x, v0, gs, gv, gl, tau, decay_input, vth, v_reset, sg, alpha, detach)
        p = tau
    xr = x if path == "replay" else None
    out = hip_backward(K, kind, gs, gv, gl, ref["h_seq"], v0, p, decay_input, vth, v_reset, detach, no.SG_IDS[sg], alpha,
                       x=xr)
    torch.testing.assert_close(out[0], ref["grad_x"], rtol=GRAD_RTOL, atol=GRAD_ATOL)
    torch.testing.assert_close(out[1], ref["grad_v_init"], rtol=GRAD_RTOL, atol=GRAD_ATOL)
    if kind == "plif":
        # float64 reference for the 10^5-term sum
        ref64 = no.forward_backward("plif_k", x.double(), v0.double(), gs.double(), gv.double(), gl.double(),
                                    kt.double(), decay_input, vth, v_reset, sg, alpha, detach)
        if torch.equal(ref64["spike_seq"].float(), ref["spike_seq"]):
            assert float(out[2]) == pytest.approx(float(ref64["grad_p"]), rel=1e-4, abs=1e-3)
        out_atomic = hip_backward(K, kind, gs, gv, gl, ref["h_seq"], v0, p, decay_input, vth, v_reset, detach,
                                  no.SG_IDS[sg], alpha, flags=_flags(atomic=True), x=xr)
        assert float(out_atomic[2]) == pytest.approx(float(out[2]), rel=1e-4, abs=1e-3)


@pytest.mark.parametrize("sg", no.SG_NAMES)
@pytest.mark.parametrize("path", ["h_seq", "replay"])
def test_backward_every_surrogate(K, sg, path):
    T, N, tau, vth = 6, 2048, 2.0, 1.0
    alpha = no.SG_DEFAULT_ALPHA[sg]
    x = seeded_randn((T, N), 700, 0.5, 1.0)
    v0 = torch.zeros(N)
    gs = seeded_randn((T, N), 701)
    ref = no.forward_backward("lif", x, v0, gs, None, None, tau, True, vth, 0.0, sg, alpha, False)
    out = hip_backward(K, "lif", gs, None, None, ref["h_seq"], v0, tau, True, vth, 0.0, False, no.SG_IDS[sg], alpha,
                       x=x if path == "replay" else None)
    torch.testing.assert_close(out[0], ref["grad_x"], rtol=GRAD_RTOL, atol=GRAD_ATOL)
    torch.testing.assert_close(out[1], ref["grad_v_init"], rtol=GRAD_RTOL, atol=GRAD_ATOL)


@pytest.mark.parametrize("which", ["none", "last", "seq", "both"])
@pytest.mark.parametrize("path", ["h_seq", "replay"])
def test_backward_grad_v_variants(K, which, path):
    T, N = 9, 1024
    x = seeded_randn((T, N), 710, 0.5, 1.0)
    v0 = seeded_randn((N,), 711, 0, 0.2)
    gs = seeded_randn((T, N), 712)
    gv = seeded_randn((T, N), 713) if which in ("seq", "both") else None
    gl = seeded_randn((N,), 714) if which in ("last", "both") else None
    ref = no.forward_backward("lif", x, v0, gs, gv, gl, 2.0, True, 1.0, 0.0, "atan", 2.0, False)
    out = hip_backward(K, "lif", gs, gv, gl, ref["h_seq"], v0, 2.0, True, 1.0, 0.0, False, 1, 2.0,
                       x=x if path == "replay" else None)
    torch.testing.assert_close(out[0], ref["grad_x"], rtol=GRAD_RTOL, atol=GRAD_ATOL)
    torch.testing.assert_close(out[1], ref["grad_v_init"], rtol=GRAD_RTOL, atol=GRAD_ATOL)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kind", ["if", "lif", "plif"])
@pytest.mark.parametrize("v_reset", [0.0, None])
@pytest.mark.parametrize("path", ["h_seq", "replay"])
def test_backward_half_storage(K, dtype, kind, v_reset, path):
    """16-bit storage: the kernel sees h_seq and the upstream gradients rounded to 16 bits.  Expected
    values come from the float64 recurrence fed exactly those rounded tensors (a spike decided on the
    rounded h is the spike the backward must use), so what is left is fp32 arithmetic plus one final
    rounding of grad_x to 16 bits: well inside the 1e-2 bar."""
    from oracle import bptt_oracle

    T, N, k, vth = 8, 4096, 0.5, 1.0
    x = seeded_randn((T, N), 720, 0.3, 1.0).to(dtype)
    v0 = seeded_randn((N,), 722, 0.0, 0.2).to(dtype)
    gs = seeded_randn((T, N), 721).to(dtype)
    gl = seeded_randn((N,), 723, 0.0, 0.1).to(dtype)
    _, _, h, raw_h = no.multi_step_mixed_precision(kind, x.float(), v0.float(), dtype, k, True, vth, v_reset,
                                                   return_raw_h=True)
    # the h_seq path sees h rounded to 16 bits, the replay path recomputes the forward's unrounded fp32 h
    h64 = (h if path == "h_seq" else raw_h).double().numpy()
    s64 = (h64 >= vth).astype(np.float64)
    vr = 0.0 if v_reset is None else v_reset
    v64 = h64 - s64 * vth if v_reset is None else s64 * vr + (1 - s64) * h64
    v_prev = np.concatenate([v0.double().numpy()[None], v64[:-1]])
    x_implied = (h64 - v_prev) / k + (v_prev - vr)  # makes the oracle's dh/dk equal (h_t - v_{t-1})/k
    sgp = lambda z: no.surrogate_grad("sigmoid", torch.from_numpy(np.ascontiguousarray(z)), 4.0).numpy()
    egx, egvi, egk = bptt_oracle.bptt(kind, h64, s64, sgp, gs.double().numpy(), None, gl.double().numpy(),
                                      0.0 if kind == "if" else k, True, vth, v_reset, False, v_prev, x_implied)
    p = {"if": 0.0, "lif": 1.0 / k, "plif": k}[kind]
    out = hip_backward(K, kind, gs, None, gl, h.to(dtype), v0, p, True, vth, v_reset, False, 0, 4.0,
                       flags=_flags(fp32_state=True), x=x if path == "replay" else None)
    assert out[0].dtype == dtype and out[1].dtype == dtype
    torch.testing.assert_close(out[0].double(), torch.from_numpy(egx), rtol=HALF_RTOL, atol=1e-3)
    torch.testing.assert_close(out[1].double(), torch.from_numpy(egvi), rtol=HALF_RTOL, atol=1e-3)
    if kind == "plif":
        assert float(out[2]) == pytest.approx(egk, rel=1e-4)


@pytest.mark.parametrize("path", ["h_seq", "replay"])
def test_plif_reduction_is_deterministic_and_accurate(K, path):
    T, N, k = 8, 1 << 18, 0.5
    x = seeded_randn((T, N), 730, 0.2, 1.0)
    v0 = torch.zeros(N)
    gs = seeded_randn((T, N), 731)
    ref = no.forward_backward("plif_k", x.double(), v0.double(), gs.double(), None, None, torch.tensor(k).double(),
                              True, 1.0, None, "sigmoid", 4.0, False)
    h = ref["h_seq"].float()
    xr = x if path == "replay" else None
    a = hip_backward(K, "plif", gs, None, None, h, v0, k, True, 1.0, None, False, 0, 4.0, x=xr)
    b = hip_backward(K, "plif", gs, None, None, h, v0, k, True, 1.0, None, False, 0, 4.0, x=xr)
    assert bits_equal(a[2], b[2])
    assert float(a[2]) == pytest.approx(float(ref["grad_p"]), rel=1e-5)


# ------------------------------------------------------------------------------------------------
# constant initial state passed as one broadcast element; optional grad_v_init
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("kind", ["if", "lif", "plif"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("recompute,T,N", [(False, 5, 64), (True, 5, 64), (False, 3, 37)])  # replay: N % 8 == 0
def test_broadcast_initial_state_equals_a_filled_tensor(K, kind, dtype, recompute, T, N):
    """An expanded one-element v_init (what a node passes while its state is the scalar reset value) must
    give bit-identical outputs and gradients to the same value filled into an [N] tensor, on the 128-bit and
    on the element-wise kernels, with h_seq saved or replayed."""
    x = seeded_randn((T, N), 41, 0.4, 1.0).to(dtype).cuda()
    gs = seeded_randn((T, N), 42).to(dtype).cuda()
    full = torch.full((N,), -0.25, dtype=dtype, device="cuda")
    bcast = torch.full((1,), -0.25, dtype=dtype, device="cuda").expand(N)
    assert bcast.stride() == (0,)
    k = torch.tensor(0.5, device="cuda")
    res = []
    for v0 in (full, bcast):
        xi = x.clone().requires_grad_()
        ki = k.clone().requires_grad_()
        if kind == "if":
            out = K.hip_multistep_if_forward(xi, v0, 0.8, -0.25, False, False, 1, 2.0, True, 0, recompute)
        elif kind == "lif":
            out = K.hip_multistep_lif_forward(xi, v0, 0.8, -0.25, False, False, 2.0, True, 1, 2.0, True, 0, recompute)
        else:
            out = K.hip_multistep_plif_forward(xi, v0, ki, 0.8, -0.25, False, False, True, 1, 2.0, True, 0, recompute)
        (out[0] * gs).sum().backward()
        res.append((out[0].detach(), out[1].detach(), out[2].detach(), xi.grad, ki.grad))
    for a, b in zip(*res):
        if a is None:
            assert b is None
        else:
            assert bits_equal(a, b)


def test_grad_v_init_is_produced_only_when_asked(K):
    x = seeded_randn((6, 128), 43, 0.4, 1.0).cuda().requires_grad_()
    v0 = seeded_randn((128,), 44, 0.0, 0.3).cuda()
    gs = seeded_randn((6, 128), 45).cuda()
    # state without requires_grad: the backward op is called with need_grad_v_init=False and returns no [N] tensor
    s = K.hip_multistep_lif_forward(x, v0, 1.0, 0.0, False, False, 2.0, True, 1, 2.0, False, 0, True)[0]
    (s * gs).sum().backward()
    gx_plain = x.grad.clone()
    x.grad = None
    v1 = v0.clone().requires_grad_()
    s = K.hip_multistep_lif_forward(x, v1, 1.0, 0.0, False, False, 2.0, True, 1, 2.0, False, 0, True)[0]
    (s * gs).sum().backward()
    assert bits_equal(x.grad, gx_plain) and v1.grad is not None and v1.grad.shape == (128,)
    gx, gvi = K.hip_multistep_lif_backward(gs, None, None, None, x.detach(), v0, 1.0, 0.0, False, False, 2.0, True, 1, 2.0,
                                           0, False)
    assert gvi.numel() == 0 and bits_equal(gx, gx_plain)
    gx, gvi = K.hip_multistep_lif_backward(gs, None, None, None, x.detach(), v0, 1.0, 0.0, False, False, 2.0, True, 1, 2.0,
                                           0, True)
    assert bits_equal(gvi, v1.grad)


@pytest.mark.parametrize("kind", ["lif", "plif"])
@pytest.mark.parametrize("decay_input", [True, False])
def test_fp16_every_op_rounding_with_a_factor_that_is_not_a_half(K, kind, decay_input):
    """fp16 storage, every op rounded, multiplying by an fp32 scalar that fp16 cannot hold (k = fl(1/3)): torch
    rounds the fp32 product to fp32 and then to fp16.  A fused mixed-precision multiply would round once and differ
    in a few percent of the elements, so the kernels must reproduce the two roundings."""
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    T, N = 6, 8192
    x = seeded_randn((T, N), 61, 0.4, 1.0).half()
    v0 = seeded_randn((N,), 62, 0.0, 0.5).half()
    k = torch.tensor(1.0 / 3.0, dtype=torch.float32)
    es, ev, eh = no.multi_step("plif_k", x, v0, k, decay_input, 0.8, -0.2)
    if kind == "plif":
        s, v, vl, h = hip_forward(K, "plif", x, v0, float(k), decay_input, 0.8, -0.2)
    else:  # LIF told to multiply by fl(1/tau) like the reference's kernels
        s, v, vl, h = hip_forward(K, "lif", x, v0, 3.0, decay_input, 0.8, -0.2, flags=L.FLAG_RECIPROCAL_TAU)
    assert bits_equal(h, eh) and bits_equal(s, es) and bits_equal(v, ev)
