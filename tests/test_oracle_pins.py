"""Pins the CPU oracle (oracle/) before anything is compared against it.

Each test is chosen so that a plausible mistake in the restatement -- a dropped term, a wrong sign
or index, a multiplication where the reference divides -- fails it.  None of these tests retypes
the oracle's own formula: expectations come from exact rational arithmetic (golden fixture),
closed forms, finite differences, numpy library routines or an independent implementation.
"""

import math

import numpy as np
import pytest
import torch

from oracle import bitpack_oracle, bptt_oracle
from oracle import neuron_oracle as no

from helpers import bits_equal, load_dyadic, seeded_randn

torch.set_num_threads(4)


# ------------------------------------------------------------------------------------------------
# 1. known-answer vectors (exact rational arithmetic), reference input test_triton_neuron.py:1207-1216
# ------------------------------------------------------------------------------------------------
def _dyadic_cases():
    doc = load_dyadic()
    return [(doc, i) for i in range(len(doc["cases"]))]


@pytest.mark.parametrize("doc,i", _dyadic_cases(), ids=lambda v: str(v) if isinstance(v, int) else "d")
def test_torch_oracle_matches_dyadic_golden(doc, i):
    c = doc["cases"][i]
    x = torch.tensor(doc["x"], dtype=torch.float32) * c["scale"]
    v0 = torch.tensor(doc["v_init"], dtype=torch.float32)
    kind = c["kind"]
    p = {"if": None, "lif": 1.0 / c["k"], "plif": torch.tensor(math.log(c["k"] / (1 - c["k"])))}[kind]
    s, v, h = no.multi_step(kind, x, v0, p, c["decay_input"], c["v_threshold"], c["v_reset"])
    assert torch.equal(s, torch.tensor(c["spike"], dtype=torch.float32))
    assert torch.equal(h, torch.tensor(c["h"], dtype=torch.float32))
    assert torch.equal(v, torch.tensor(c["v"], dtype=torch.float32))


@pytest.mark.parametrize("doc,i", _dyadic_cases(), ids=lambda v: str(v) if isinstance(v, int) else "d")
def test_c_oracle_matches_dyadic_golden(doc, i, c_oracle):
    c = doc["cases"][i]
    x = np.array(doc["x"], dtype=np.float32) * np.float32(c["scale"])
    v0 = np.array(doc["v_init"], dtype=np.float32)
    tau = {"if": 1.0, "lif": 1.0 / c["k"], "plif": c["k"]}[c["kind"]]
    s, v, h = c_oracle.forward_f32(c["kind"], x, v0, tau, c["decay_input"], c["v_threshold"], c["v_reset"])
    assert np.array_equal(s, np.array(c["spike"], dtype=np.float32))
    assert np.array_equal(h, np.array(c["h"], dtype=np.float32))
    assert np.array_equal(v, np.array(c["v"], dtype=np.float32))


@pytest.mark.parametrize("storage", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("doc,i", _dyadic_cases(), ids=lambda v: str(v) if isinstance(v, int) else "d")
def test_half_precision_oracles_match_dyadic_golden(doc, i, storage):
    """All golden values fit bf16, so both 16-bit semantics must reproduce them exactly."""
    c = doc["cases"][i]
    x = torch.tensor(doc["x"], dtype=torch.float32) * c["scale"]
    v0 = torch.tensor(doc["v_init"], dtype=torch.float32)
    kind = c["kind"]
    for order in (True, False):
        if not order and c["v_reset"] not in (0.0, None):
            continue
        s, v, h = no.multi_step_mixed_precision(kind, x, v0, storage, c["k"], c["decay_input"], c["v_threshold"],
                                                c["v_reset"], torch_op_order=order)
        assert torch.equal(s, torch.tensor(c["spike"], dtype=torch.float32))
        assert torch.equal(h, torch.tensor(c["h"], dtype=torch.float32))
        assert torch.equal(v, torch.tensor(c["v"], dtype=torch.float32))
    p = {"if": None, "lif": 1.0 / c["k"], "plif": torch.tensor(math.log(c["k"] / (1 - c["k"])))}[kind]
    s, v, h = no.multi_step(kind, x.to(storage), v0.to(storage), p, c["decay_input"], c["v_threshold"], c["v_reset"])
    assert s.dtype == storage and v.dtype == storage
    assert torch.equal(s.float(), torch.tensor(c["spike"], dtype=torch.float32))
    assert torch.equal(v.float(), torch.tensor(c["v"], dtype=torch.float32))


# ------------------------------------------------------------------------------------------------
# 2. closed forms and invariants
# ------------------------------------------------------------------------------------------------
def test_single_step_from_rest_is_x_over_tau():
    x = seeded_randn((1, 1000), 1)
    for tau in (2.0, 3.0, 10.0):
        _, _, h = no.multi_step("lif", x, torch.zeros(1000), tau, True, 1e9, 0.0)
        assert torch.equal(h[0], x[0] / tau)
        _, _, h = no.multi_step("lif", x, torch.zeros(1000), tau, False, 1e9, 0.0)
        assert torch.equal(h[0], x[0])


def test_zero_input_decays_geometrically_towards_v_reset():
    T, tau, vr = 12, 4.0, -0.5
    v0 = torch.tensor([0.75, -1.25, 0.0], dtype=torch.float64)
    x = torch.zeros(T, 3, dtype=torch.float64)
    for decay_input in (True, False):
        _, v, h = no.multi_step("lif", x, v0, tau, decay_input, 10.0, vr)
        expect = torch.stack([vr + (v0 - vr) * (1 - 1 / tau) ** (t + 1) for t in range(T)])
        torch.testing.assert_close(h, expect, rtol=1e-13, atol=1e-13)
        torch.testing.assert_close(v, expect, rtol=1e-13, atol=1e-13)


def test_if_soft_reset_rate_coding_identity():
    """Constant dyadic input x in [0,1), v_th=1, soft reset: after T steps the spike count is
    floor(T x) and the residual potential is T x - count, exactly (ANN2SNN rate coding)."""
    T = 32
    xs = torch.arange(0, 64, dtype=torch.float32) / 64.0
    x = xs.expand(T, -1).contiguous()
    s, v, _ = no.multi_step("if", x, torch.zeros(64), None, True, 1.0, None)
    count = s.sum(0)
    assert torch.equal(count, torch.floor(T * xs))
    assert torch.equal(v[-1], T * xs - count)
    # the same in fp16 (all values exact there too)
    s16, v16, _ = no.multi_step("if", x.half(), torch.zeros(64).half(), None, True, 1.0, None)
    assert torch.equal(s16.float(), s) and torch.equal(v16.float(), v)


@pytest.mark.parametrize("kind,p", [("if", None), ("lif", 3.0), ("plif", torch.tensor(0.3))])
@pytest.mark.parametrize("v_reset", [0.0, -0.2, None])
def test_fire_and_reset_invariants(kind, p, v_reset):
    x = seeded_randn((9, 500), 7, 0.4, 1.0)
    vth = 0.8
    s, v, h = no.multi_step(kind, x, torch.zeros(500), p, True, vth, v_reset)
    assert set(s.unique().tolist()) <= {0.0, 1.0}
    assert torch.equal(s, (h >= vth).float())
    fired = s.bool()
    assert fired.any() and (~fired).any()
    if v_reset is None:
        assert torch.equal(v[fired], h[fired] - vth)
    else:
        assert torch.equal(v[fired], torch.full_like(v[fired], v_reset))
    assert torch.equal(v[~fired], h[~fired])


def test_plif_equals_lif_when_tau_is_a_power_of_two():
    """k = sigmoid(-log(tau-1)) = 1/tau; for tau = 2 the product equals the quotient bit for bit."""
    x = seeded_randn((8, 777), 11, 0.3, 0.8)
    w = torch.tensor(-math.log(2.0 - 1.0))
    for decay_input in (True, False):
        a = no.multi_step("lif", x, torch.zeros(777), 2.0, decay_input, 1.0, 0.0)
        b = no.multi_step("plif", x, torch.zeros(777), w, decay_input, 1.0, 0.0)
        for u, w_ in zip(a, b):
            assert bits_equal(u, w_)


def test_lif_divides_rather_than_multiplies():
    """The torch backend divides by tau; a restatement that multiplies by 1/tau differs for tau=3."""
    x = seeded_randn((1, 100000), 5)
    _, _, h = no.multi_step("lif", x, torch.zeros(100000), 3.0, True, 1e9, 0.0)
    assert torch.equal(h[0], x[0] / 3.0)
    assert not torch.equal(h[0], x[0] * (1.0 / 3.0))


# ------------------------------------------------------------------------------------------------
# 3. surrogate gradients: finite difference of the primitive (reference
#    test_neuron_kernel_surrogate_contract.py:25-44) and the values at 0
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["sigmoid", "atan", "piecewise_quadratic", "piecewise_exp", "soft_sign", "erf"])
def test_surrogate_gradient_is_derivative_of_primitive(name):
    alpha = no.SG_DEFAULT_ALPHA[name]
    x = torch.tensor([-0.75, -0.25, 0.25, 0.75], dtype=torch.float64)
    xs = x.clone().requires_grad_()
    out = no.surrogate(name, alpha)(xs)
    out.sum().backward()
    eps = 1e-5
    fd = (no.primitive(name, x + eps, alpha) - no.primitive(name, x - eps, alpha)) / (2 * eps)
    assert torch.equal(out.detach(), no.heaviside(x))
    torch.testing.assert_close(xs.grad, fd, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(no.surrogate_grad(name, x, alpha), fd, atol=1e-4, rtol=1e-4)


def test_surrogate_gradient_values_at_zero():
    z = torch.zeros(1, dtype=torch.float64)
    assert no.surrogate_grad("atan", z, 2.0).item() == pytest.approx(1.0)        # alpha/2
    assert no.surrogate_grad("atan", z, 3.0).item() == pytest.approx(1.5)
    assert no.surrogate_grad("sigmoid", z, 4.0).item() == pytest.approx(1.0)     # alpha/4
    assert no.surrogate_grad("super_spike", z, 1.5).item() == pytest.approx(1.5)  # alpha
    assert no.surrogate_grad("erf", z, 2.0).item() == pytest.approx(2.0 / math.sqrt(math.pi))


def test_super_spike_gradient_away_from_zero():
    """alpha / (|x| + 1)^2 (surrogate.py:1101-1102; the reference defines no primitive to difference, :1236-1237):
    hand-computed values, exact in binary floating point."""
    x = torch.tensor([1.0, -3.0, 0.5, -0.25], dtype=torch.float64)
    want = torch.tensor([2.0 / 4.0, 2.0 / 16.0, 2.0 / 2.25, 2.0 / 1.5625], dtype=torch.float64)
    assert torch.equal(no.surrogate_grad("super_spike", x, 2.0), want)
    xs = x.clone().requires_grad_()
    g = torch.tensor([1.0, -2.0, 0.5, 4.0], dtype=torch.float64)
    no.surrogate("super_spike", 2.0)(xs).backward(g)
    assert torch.equal(xs.grad, want * g)


def test_reciprocal_tau_form_is_a_multiplication_by_the_rounded_reciprocal():
    """What the reference's kernel backends and torch on a GPU compute for the LIF charge (multi_step/lif.py:338 passes
    `reciprocal_tau`; a division of a device tensor by a Python scalar runs as a multiplication by 1/b): the oracle's
    "plif_k" charge fed k = fl32(1/tau).  Pinned against numpy float32 arithmetic written out op by op, and shown to
    differ from the IEEE division of the CPU backend for tau = 3."""
    x = seeded_randn((4096,), 77, 0.3, 1.0)
    v = seeded_randn((4096,), 78, 0.1, 0.5)
    k32 = np.float32(1.0) / np.float32(3.0)
    xn, vn, vr = x.numpy(), v.numpy(), np.float32(-0.2)
    for decay_input in (True, False):
        want = vn + (xn - (vn - vr)) * k32 if decay_input else vn - (vn - vr) * k32 + xn
        got = no.charge("plif_k", x, v, torch.tensor(float(k32)), decay_input, -0.2)
        assert want.dtype == np.float32 and np.array_equal(got.numpy(), want)
        assert not torch.equal(got, no.charge("lif", x, v, 3.0, decay_input, -0.2))
    # tau a power of two: both forms agree bit for bit
    assert torch.equal(no.charge("plif_k", x, v, torch.tensor(0.25), True, -0.2), no.charge("lif", x, v, 4.0, True, -0.2))


# ------------------------------------------------------------------------------------------------
# 4. BPTT: closed-form recurrence == autograd of the restated ops == finite differences
# ------------------------------------------------------------------------------------------------
def _np_sg_prime(name, alpha):
    return lambda z: no.surrogate_grad(name, torch.from_numpy(np.ascontiguousarray(z)), alpha).numpy()


GRID = [(kind, sg, di, vr, det)
        for kind in ("if", "lif", "plif")
        for sg in ("atan", "sigmoid")
        for di in ((True,) if kind == "if" else (True, False))
        for vr in (0.0, -0.2, None)
        for det in (False, True)]


@pytest.mark.parametrize("kind,sg,decay_input,v_reset,detach", GRID)
def test_recurrence_equals_autograd_float64(kind, sg, decay_input, v_reset, detach):
    T, N, tau, vth = 6, 257, 3.0, 0.7
    alpha = no.SG_DEFAULT_ALPHA[sg]
    x = seeded_randn((T, N), 21, 0.4, 1.0, torch.float64)
    v0 = seeded_randn((N,), 22, 0.0, 0.3, torch.float64)
    gs = seeded_randn((T, N), 23, dtype=torch.float64)
    gv = seeded_randn((T, N), 24, 0.0, 0.1, torch.float64)
    gl = seeded_randn((N,), 25, 0.0, 0.1, torch.float64)
    w = torch.tensor(-math.log(tau - 1.0), dtype=torch.float64)
    p = {"if": None, "lif": tau, "plif": w}[kind]
    ref = no.forward_backward(kind, x, v0, gs, gv, gl, p, decay_input, vth, v_reset, sg, alpha, detach)
    k = {"if": 0.0, "lif": 1.0 / tau, "plif": float(w.sigmoid())}[kind]
    v_prev = torch.cat([v0[None], ref["v_seq"][:-1]]).numpy()
    gx, gvi, gk = bptt_oracle.bptt(kind, ref["h_seq"].numpy(), ref["spike_seq"].numpy(), _np_sg_prime(sg, alpha),
                                   gs.numpy(), gv.numpy(), gl.numpy(), k, decay_input, vth, v_reset, detach,
                                   v_prev, x.numpy())
    np.testing.assert_allclose(gx, ref["grad_x"].numpy(), rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(gvi, ref["grad_v_init"].numpy(), rtol=1e-11, atol=1e-13)
    if kind == "plif":
        # dL/dw = dL/dk * k (1 - k)   (reference test_triton_neuron.py:807-809)
        assert gk * k * (1 - k) == pytest.approx(float(ref["grad_p"]), rel=1e-10)


@pytest.mark.parametrize("kind,decay_input", [("if", True), ("lif", True), ("lif", False), ("plif", True), ("plif", False)])
@pytest.mark.parametrize("v_reset", [0.0, -0.2, None])
def test_recurrence_matches_finite_differences_of_the_smooth_network(kind, v_reset, decay_input):
    """With the primitive (non-spiking) surrogate the network is smooth, autograd is its true
    gradient and the recurrence (s_t = primitive, sg = primitive') must match central differences."""
    T, N, tau, vth, alpha = 5, 7, 2.5, 0.6, 2.0
    x = seeded_randn((T, N), 31, 0.4, 0.8, torch.float64)
    v0 = seeded_randn((N,), 32, 0.0, 0.3, torch.float64)
    gs = seeded_randn((T, N), 33, dtype=torch.float64)
    gv = seeded_randn((T, N), 34, dtype=torch.float64)
    w = torch.tensor(-math.log(tau - 1.0), dtype=torch.float64)
    p = {"if": None, "lif": tau, "plif": w}[kind]
    k = {"if": 0.0, "lif": 1.0 / tau, "plif": float(w.sigmoid())}[kind]
    smooth = no.surrogate("atan", alpha, spiking=False)

    def loss(x_, v0_, k_=None):
        pp = p if k_ is None else k_
        kk = kind if k_ is None else "plif_k"
        s, v, _ = no.multi_step(kk, x_, v0_, pp, decay_input, vth, v_reset, smooth)
        return float((s * gs).sum() + (v * gv).sum())

    s, v, h = no.multi_step(kind, x, v0, p, decay_input, vth, v_reset, smooth)
    v_prev = torch.cat([v0[None], v[:-1]]).numpy()
    gx, gvi, gk = bptt_oracle.bptt(kind, h.numpy(), s.numpy(), _np_sg_prime("atan", alpha), gs.numpy(), gv.numpy(),
                                   None, k, decay_input, vth, v_reset, False, v_prev, x.numpy())
    eps = 1e-6
    for (t, n) in [(0, 0), (2, 3), (T - 1, N - 1)]:
        xp, xm = x.clone(), x.clone()
        xp[t, n] += eps
        xm[t, n] -= eps
        assert (loss(xp, v0) - loss(xm, v0)) / (2 * eps) == pytest.approx(gx[t, n], rel=1e-6, abs=1e-8)
    vp, vm = v0.clone(), v0.clone()
    vp[2] += eps
    vm[2] -= eps
    assert (loss(x, vp) - loss(x, vm)) / (2 * eps) == pytest.approx(gvi[2], rel=1e-6, abs=1e-8)
    if kind == "plif":
        kt = torch.tensor(k, dtype=torch.float64)
        fd = (loss(x, v0, kt + eps) - loss(x, v0, kt - eps)) / (2 * eps)
        assert fd == pytest.approx(gk, rel=1e-6, abs=1e-8)


def test_c_backward_equals_recurrence(c_oracle):
    T, N, tau, vth = 7, 129, 3.0, 0.9
    x = seeded_randn((T, N), 41, 0.4, 1.0)
    v0 = seeded_randn((N,), 42, 0.0, 0.3)
    gs, gv, gl = seeded_randn((T, N), 43), seeded_randn((T, N), 44, 0, 0.1), seeded_randn((N,), 45, 0, 0.1)
    for kind in ("if", "lif", "plif"):
        for sg_id, sg in enumerate(no.SG_NAMES):
            for v_reset in (0.0, -0.2, None):
                for detach in (False, True):
                    for di in ((True,) if kind == "if" else (True, False)):
                        k = 0.0 if kind == "if" else 1.0 / tau
                        alpha = no.SG_DEFAULT_ALPHA[sg]
                        s, v, h = c_oracle.forward_f32(kind, x.numpy(), v0.numpy(), tau if kind == "lif" else k, di,
                                                       vth, v_reset)
                        v_prev = np.concatenate([v0.numpy()[None], v[:-1]]).astype(np.float64)
                        e = bptt_oracle.bptt(kind, h, s, _np_sg_prime(sg, alpha), gs.double().numpy(),
                                             gv.double().numpy(), gl.double().numpy(), float(np.float32(k)) if kind == "plif" else k,
                                             di, vth, v_reset, detach, v_prev, x.double().numpy())
                        a = c_oracle.backward_f64(kind, gs.numpy(), gv.numpy(), gl.numpy(), h,
                                                  float(np.float32(k)) if kind == "plif" else k, di, vth, v_reset,
                                                  detach, sg_id, alpha, x.numpy(), v0.numpy(), v)
                        np.testing.assert_allclose(a[0], e[0], rtol=1e-9, atol=1e-12)
                        np.testing.assert_allclose(a[1], e[1], rtol=1e-9, atol=1e-12)
                        if kind == "plif":
                            assert a[2] == pytest.approx(e[2], rel=1e-9)


# ------------------------------------------------------------------------------------------------
# 5. torch oracle == C oracle bit for bit (two independent implementations of IEEE fp32)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("kind,decay_input,tau", [("if", True, 2.0)] + [(kind, di, tau) for kind in ("lif", "plif")
                                                  for di in (True, False) for tau in (2.0, 3.0, 10.0)])
@pytest.mark.parametrize("v_reset", [0.0, -0.2, None])
def test_torch_and_c_oracle_agree_bitwise(kind, v_reset, decay_input, tau, c_oracle):
    T, N = 16, 4099
    x = seeded_randn((T, N), 51, 0.3, 0.8)
    v0 = seeded_randn((N,), 52, 0.0, 0.2)
    if kind == "plif":
        w = torch.tensor(-math.log(tau - 1.0))
        kf = float(w.sigmoid())  # the fp32 value torch multiplies by
        s, v, h = no.multi_step("plif", x, v0, w, decay_input, 0.5, v_reset)
        cs, cv, ch = c_oracle.forward_f32("plif", x.numpy(), v0.numpy(), kf, decay_input, 0.5, v_reset)
    else:
        s, v, h = no.multi_step(kind, x, v0, tau, decay_input, 0.5, v_reset)
        cs, cv, ch = c_oracle.forward_f32(kind, x.numpy(), v0.numpy(), tau, decay_input, 0.5, v_reset)
    assert 0.001 < s.mean() < 0.7
    assert bits_equal(s, torch.from_numpy(cs))
    assert bits_equal(h, torch.from_numpy(ch))
    assert bits_equal(v, torch.from_numpy(cv))


# ------------------------------------------------------------------------------------------------
# 6. bit-packing
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [0, 1, 6, 7, 8, 9, 17, 64, 1000, 4097])
def test_bitpack_oracles_equal_numpy_packbits(n, c_oracle):
    rng = np.random.default_rng(n)
    bits = (rng.random(n) < 0.3).astype(np.float32)
    expect = np.packbits(bits.astype(np.uint8), bitorder="little")
    got = bitpack_oracle.bit_spike_compress(bits)
    assert np.array_equal(got, expect)
    assert np.array_equal(c_oracle.bit_pack(bits), expect)
    assert np.array_equal(bitpack_oracle.bit_spike_decompress(got, (n,)), bits.astype(np.uint8))
    assert np.array_equal(c_oracle.bit_unpack(got, n), bits.astype(np.uint8))
    assert np.array_equal(np.unpackbits(got, bitorder="little")[:n], bits.astype(np.uint8))


def test_bitpack_reference_round_trips(c_oracle):
    # test/activation_based/test_checkpointing.py:275-282 and :647-662
    spikes = np.array([[1.0, 0.0, 1.0], [0.0, 1.0, 0.0]], dtype=np.float32)
    packed = bitpack_oracle.bit_spike_compress(spikes)
    assert packed.tolist() == [0b010101]
    assert np.array_equal(bitpack_oracle.bit_spike_decompress(packed, spikes.shape), spikes.astype(np.uint8))
    # test/activation_based/test_cuda_custom_op_migration.py:179-190: 17 elements, every third one set
    spike = (np.arange(17) % 3 == 0).astype(np.float32)
    packed = bitpack_oracle.bit_spike_compress(spike)
    assert packed.tolist() == [0b01001001, 0b10010010, 0b0]
    assert np.array_equal(c_oracle.bit_pack(spike), packed)
    assert np.array_equal(bitpack_oracle.bit_spike_decompress(packed, (17,)), spike.astype(np.uint8))


def test_bitpack_nonzero_semantics(c_oracle):
    """`.to(torch.bool)`: -0.0 is no spike, NaN / 2.0 / subnormals are."""
    vals = np.array([0.0, -0.0, 1.0, 2.0, np.nan, 1e-45, -1.0, 0.0], dtype=np.float32)
    expect = np.packbits(torch.from_numpy(vals).to(torch.bool).numpy().astype(np.uint8), bitorder="little")
    assert np.array_equal(bitpack_oracle.bit_spike_compress(vals), expect)
    assert np.array_equal(c_oracle.bit_pack(vals), expect)
    for dt in (torch.float16, torch.bfloat16):
        t = torch.from_numpy(vals).to(dt)
        e = np.packbits(t.to(torch.bool).numpy().astype(np.uint8), bitorder="little")
        assert np.array_equal(c_oracle.bit_pack(t.view(torch.int16).numpy()), e)


# ------------------------------------------------------------------------------------------------
# 7. spiking self-attention contraction
# ------------------------------------------------------------------------------------------------
def test_ssa_oracle_is_exact_and_associative():
    """(V K^T) Q == V (K^T Q) in integers; all-ones input has the closed form scale * L * Cph; the float
    restatement equals the integer one because every partial sum is an integer below 2^24."""
    from oracle import ssa_oracle

    g = torch.Generator().manual_seed(3)
    qkv = (torch.rand((5, 3, 4, 32, 50), generator=g) < 0.3).float()
    exact = ssa_oracle.ssa_exact(qkv, 0.125)
    q, k, v = (qkv[:, i].to(torch.int64) for i in range(3))
    other_order = (v @ (k.transpose(-2, -1) @ q)).double() * 0.125
    assert torch.equal(exact, other_order)
    assert torch.equal(ssa_oracle.ssa(qkv, 0.125).double(), exact)
    ones = torch.ones(1, 3, 2, 8, 11)
    assert torch.equal(ssa_oracle.ssa_exact(ones, 0.125), torch.full((1, 2, 8, 11), 0.125 * 11 * 8, dtype=torch.float64))
    # a single spike in v[c1, l0], k[c2, l0], q[c2, l1] lights out[c1, l1] only
    one = torch.zeros(1, 3, 1, 4, 6)
    one[0, 2, 0, 1, 3] = 1  # v
    one[0, 1, 0, 2, 3] = 1  # k
    one[0, 0, 0, 2, 5] = 1  # q
    out = ssa_oracle.ssa_exact(one, 1.0)
    assert out[0, 0, 1, 5] == 1 and out.sum() == 1


# ------------------------------------------------------------------------------------------------
# QIF (functional/neuron.py:397): pins that do not retype the formula
# ------------------------------------------------------------------------------------------------
def test_qif_rest_and_critical_potentials_are_fixed_points_without_input():
    """With x = 0 the quadratic term vanishes at v = v_rest and v = v_c, so both are fixed points of the charge
    step; between them the potential falls towards v_rest, above v_c it escapes upwards (the defining property of
    the quadratic integrate-and-fire model)."""
    tau, a0, v_rest, v_c = 2.0, 1.0, 0.0, 0.5
    p = (tau, a0, v_rest, v_c)
    zeros = torch.zeros(1, 4)
    v0 = torch.tensor([v_rest, v_c, 0.25, 0.75])
    _, v, h = no.multi_step("qif", zeros, v0, p, True, 10.0, -0.1)
    assert float(h[0, 0]) == v_rest and float(h[0, 1]) == v_c
    assert float(h[0, 2]) < 0.25 and float(h[0, 3]) > 0.75
    # 0.25 -> 0.25 + (0.25)(-0.25)/2 exactly (all dyadic)
    assert float(h[0, 2]) == 0.25 - 0.03125
    assert float(h[0, 3]) == 0.75 + 0.09375


def test_qif_single_step_closed_form_and_reduction_to_if():
    """T = 1 from v = 0: h = (x + a0 v_rest v_c) / tau.  A vanishing a0 leaves h = v + x / tau, i.e. an IF neuron
    driven by x / tau."""
    x = seeded_randn((1, 64), 11, 0.5, 1.0)
    v0 = torch.zeros(64)
    _, _, h = no.multi_step("qif", x, v0, (4.0, 2.0, 0.25, 0.5), True, 100.0, None)
    assert torch.equal(h[0], (x[0] + 0.25) / 4.0)  # a0 v_rest v_c = 2 * 0.25 * 0.5
    xs = seeded_randn((6, 64), 12, 0.5, 1.0)
    s_q, v_q, _ = no.multi_step("qif", xs, v0, (2.0, 0.0, 0.0, 0.5), True, 1.0, 0.0)
    s_i, v_i, _ = no.multi_step("if", xs / 2.0, v0, None, True, 1.0, 0.0)
    assert torch.equal(s_q, s_i) and torch.equal(v_q, v_i)


@pytest.mark.parametrize("v_reset", [-0.1, None])
def test_qif_autograd_matches_finite_differences_of_the_smooth_network(v_reset):
    T, N, vth, alpha = 5, 6, 0.9, 2.0
    p = (2.5, 1.3, 0.0, 0.6)
    x = seeded_randn((T, N), 41, 0.4, 0.8, torch.float64)
    v0 = seeded_randn((N,), 42, 0.0, 0.3, torch.float64)
    gs = seeded_randn((T, N), 43, dtype=torch.float64)
    gv = seeded_randn((T, N), 44, dtype=torch.float64)
    smooth = no.surrogate("atan", alpha, spiking=False)

    def loss(x_, v0_):
        s, v, _ = no.multi_step("qif", x_, v0_, p, True, vth, v_reset, smooth)
        return float((s * gs).sum() + (v * gv).sum())

    ref = no.forward_backward("qif", x, v0, gs, gv, None, p, True, vth, v_reset, "atan", alpha, False, spiking=False)
    eps = 1e-6
    for (t, n) in [(0, 0), (2, 3), (T - 1, N - 1)]:
        xp, xm = x.clone(), x.clone()
        xp[t, n] += eps
        xm[t, n] -= eps
        assert (loss(xp, v0) - loss(xm, v0)) / (2 * eps) == pytest.approx(float(ref["grad_x"][t, n]), rel=1e-6, abs=1e-8)
    vp, vm = v0.clone(), v0.clone()
    vp[2] += eps
    vm[2] -= eps
    assert (loss(x, vp) - loss(x, vm)) / (2 * eps) == pytest.approx(float(ref["grad_v_init"][2]), rel=1e-6, abs=1e-8)


# ------------------------------------------------------------------------------------------------
# ILIF (functional/neuron.py:1097-1099): the reference's own known-answer values, invariants, recurrence
# ------------------------------------------------------------------------------------------------
def _ilif(x_seq, v0, tau=4.0 / 3.0, v_th=1.0, levels=4, window=None, detach=False):
    return no.multi_step("ilif", x_seq, v0, tau, False, v_th, None, no.multi_level_spike_count(levels, window), detach)


def test_ilif_oracle_reproduces_the_reference_tests_literal_values():
    """Inputs and expected outputs of test/activation_based/test_ilif_node.py:336-344, 354-361, 364-370, 400-413."""
    s, v, _ = _ilif(torch.tensor([[3.2, 0.4, 5.8]]), torch.zeros(3))
    assert torch.equal(s, torch.tensor([[3.0, 0.0, 4.0]]))
    torch.testing.assert_close(v[0], torch.tensor([3.2, 0.4, 5.8]) - torch.tensor([3.0, 0.0, 4.0]))
    s, v, _ = _ilif(torch.tensor([[3.2], [0.0]]), torch.zeros(1))
    assert torch.equal(s[1], torch.tensor([0.0]))
    torch.testing.assert_close(v[1], torch.tensor([0.05]))  # the residual 0.2 decayed by 1 - 1/tau = 0.25
    s, v, _ = _ilif(torch.tensor([[3.2, 5.8]]), torch.zeros(2))
    assert torch.equal(s, torch.tensor([[3.0, 4.0]]))
    torch.testing.assert_close(v[0], torch.tensor([0.2, 1.8]))
    s, _, _ = _ilif(torch.tensor([[3.2], [0.0], [4.8], [0.0]]), torch.zeros(1))
    assert torch.equal(s.flatten(), torch.tensor([3.0, 0.0, 4.0, 0.0]))


def test_ilif_oracle_gradient_window_matches_the_reference_tests_literal_values():
    """test_ilif_node.py:416-440: y.sum().backward() through one step from rest."""
    x = torch.tensor([[-0.5, 0.5, 4.5]])
    r = no.forward_backward("ilif", x, torch.zeros(3), torch.ones(1, 3), None, None, 2.0, False, 1.0, None,
                            sg=no.multi_level_spike_count(4))
    assert torch.equal(r["spike_seq"], torch.tensor([[0.0, 0.0, 4.0]]))
    torch.testing.assert_close(r["grad_x"], torch.tensor([[0.0, 1.0, 0.0]]))
    x = torch.tensor([[-0.25, 4.25, 4.75]])
    r = no.forward_backward("ilif", x, torch.zeros(3), torch.ones(1, 3), None, None, 2.0, False, 1.0, None,
                            sg=no.multi_level_spike_count(4, (-0.5, 4.5)))
    assert torch.equal(r["spike_seq"], torch.tensor([[0.0, 4.0, 4.0]]))
    torch.testing.assert_close(r["grad_x"], torch.tensor([[1.0, 1.0, 0.0]]))


def test_ilif_invariants_and_reduction_to_a_soft_reset_lif():
    """Counts are integers in [0, D]; v = h - c v_th; inside the quantiser's range the residual is at most half a
    threshold; ties round to even.  With D = 1 the count is [h/v_th > 1/2]: a soft-reset LIF without input decay
    that fires above v_th/2 but is reset by v_th -- checked against that neuron written out step by step."""
    x = seeded_randn((12, 500), 71, 0.9, 1.5)
    v0 = seeded_randn((500,), 72, 0.0, 0.3)
    for v_th, levels in ((1.0, 4), (0.7, 2), (0.25, 7)):
        s, v, h = _ilif(x, v0, tau=1.6, v_th=v_th, levels=levels)
        assert bool(((s >= 0) & (s <= levels) & (s == s.round())).all()) and float(s.max()) == levels
        assert torch.equal(v, h - s * v_th)
        inside = (h / v_th >= 0) & (h / v_th <= levels)
        assert float((v[inside].abs() / v_th).max()) <= 0.5 + 1e-6
    dyadic = torch.tensor([[0.5, 1.5, 2.5, 3.5, 4.5, -0.5]])
    s, _, _ = _ilif(dyadic, torch.zeros(6))
    assert torch.equal(s, torch.tensor([[0.0, 2.0, 2.0, 4.0, 4.0, 0.0]]))

    tau, v_th = 1.6, 0.8
    s1, v1, _ = _ilif(x, v0, tau=tau, v_th=v_th, levels=1)
    v = v0
    for t in range(x.shape[0]):
        h = v - v / tau + x[t]
        fired = (h / v_th > 0.5).float()
        v = h - fired * v_th
        assert torch.equal(s1[t], fired) and torch.equal(v1[t], v)


@pytest.mark.parametrize("detach", [False, True])
@pytest.mark.parametrize("window", [None, (-0.5, 2.25)])
def test_ilif_recurrence_equals_autograd_float64(detach, window):
    T, N, tau, v_th, levels = 6, 257, 1.7, 0.6, 3
    x = seeded_randn((T, N), 81, 0.5, 1.0, torch.float64)
    v0 = seeded_randn((N,), 82, 0.0, 0.3, torch.float64)
    gs = seeded_randn((T, N), 83, dtype=torch.float64)
    gv = seeded_randn((T, N), 84, 0.0, 0.1, torch.float64)
    gl = seeded_randn((N,), 85, 0.0, 0.1, torch.float64)
    ref = no.forward_backward("ilif", x, v0, gs, gv, gl, tau, False, v_th, None, detach_reset=detach,
                              sg=no.multi_level_spike_count(levels, window))
    lo, hi = (0.0, float(levels)) if window is None else window
    gx, gvi = bptt_oracle.bptt_ilif(ref["h_seq"].numpy(), gs.numpy(), gv.numpy(), gl.numpy(), 1.0 / tau, v_th, lo, hi,
                                    detach)
    np.testing.assert_allclose(gx, ref["grad_x"].numpy(), rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(gvi, ref["grad_v_init"].numpy(), rtol=1e-11, atol=1e-13)
    z = ref["h_seq"] / v_th
    assert 0.05 < float(((z >= lo) & (z <= hi)).double().mean()) < 0.95  # both sides of the window are exercised


# ------------------------------------------------------------------------------------------------
# ST-BIF (functional/neuron.py:3234-3247): the quantiser it must reproduce, literal cases of the reference's tests
# ------------------------------------------------------------------------------------------------
def _stbif_tensors(scale, pos_max, neg_min):
    return torch.tensor(float(scale)), torch.tensor(float(pos_max)), torch.tensor(float(neg_min))


@pytest.mark.parametrize("scale,pos_max,neg_min", [(0.25, 3, -4), (0.125, 7, 0), (0.3, 1, -2)])
def test_stbif_released_total_equals_the_quantiser(scale, pos_max, neg_min):
    """Defining property (reference test_ann2snn_transformer.py:792-803 with the quantiser of :570-573): feed x once,
    then zeros; the outputs sum to  s * clamp(floor(x/s + 1/2), neg_min, pos_max)  once enough steps have run.
    Independent of the step formula: it is the closed form the neuron exists to reproduce."""
    from oracle import stbif_oracle

    x = seeded_randn((1, 400), 91, 0.0, 1.0, torch.float64)
    x[0, :4] = torch.tensor([-0.75, -0.2, 0.3, 0.9], dtype=torch.float64)
    T = 16
    x_seq = torch.cat([x, torch.zeros((T - 1, 400), dtype=torch.float64)])
    th = [t.double() for t in _stbif_tensors(scale, pos_max, neg_min)]
    scale = float(th[0])  # the fp32 value the neuron holds
    out, q, acc, cur, work = stbif_oracle.multi_step(x_seq, torch.full((400,), 0.5, dtype=torch.float64),
                                                     torch.zeros(400, dtype=torch.float64), *th)
    expected = torch.clamp(torch.floor(x[0] / scale + 0.5), neg_min, pos_max) * scale
    torch.testing.assert_close(out.sum(0), expected, rtol=0, atol=1e-12)
    assert set(torch.unique(out / scale).round().tolist()) <= {-1.0, 0.0, 1.0} and work
    assert torch.equal(acc, (expected / scale).round())
    if scale == 0.25 and pos_max == 3:  # the reference test's literal case: [-0.75, -0.2, 0.3, 0.9] -> [-0.75, -0.25, 0.25, 0.75]
        assert out.sum(0)[:4].tolist() == [-0.75, -0.25, 0.25, 0.75]


def test_stbif_rounds_the_accumulator_half_to_even_and_reports_work():
    """Literal case of the reference's test_ann2snn_transformer.py:975-1010 (x = 0, q = 1/2, half-integer acc_q) and
    of test_functional_neuron.py:690-705 (is_work)."""
    from oracle import stbif_oracle

    x = torch.zeros(6)
    acc = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, -2.5])
    out, q, acc2, cur = stbif_oracle.step(x, torch.full_like(x, 0.5), acc, *_stbif_tensors(0.1, 10, -10))
    assert torch.equal(acc2, torch.tensor([0.0, 2.0, 2.0, -0.0, -2.0, -2.0]))
    assert torch.equal(out, torch.zeros(6)) and torch.equal(q, torch.full_like(x, 0.5)) and torch.equal(cur, torch.zeros(6))
    th = _stbif_tensors(0.25, 3, -4)
    z = torch.zeros(2, 2, 3)
    assert stbif_oracle.multi_step(z, torch.full((2, 3), 0.5), torch.zeros(2, 3), *th)[4] is False
    z[1] = 0.25
    assert stbif_oracle.multi_step(z, torch.full((2, 3), 0.5), torch.zeros(2, 3), *th)[4] is True


def test_stbif_bounds_block_release_and_both_arithmetic_forms_agree_in_fp32():
    """A saturated accumulator stops releasing in that direction while the residual keeps integrating; the Triton
    kernel's form (q >= 1, q - pos + neg) equals the torch form in fp32."""
    from oracle import stbif_oracle

    th = _stbif_tensors(0.5, 2, -1)
    x_seq = torch.full((8, 1), 1.0)  # two units per step
    out, q, acc, cur, _ = stbif_oracle.multi_step(x_seq, torch.full((1,), 0.5), torch.zeros(1), *th)
    assert out.flatten().tolist() == [0.5, 0.5, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0] and float(acc) == 2.0
    assert float(q) == 0.5 + 16 - 2
    x = seeded_randn((20, 300), 92, 0.0, 0.6)
    a = stbif_oracle.multi_step(x, torch.full((300,), 0.5), torch.zeros(300), *_stbif_tensors(0.25, 3, -4))
    b = stbif_oracle.multi_step_fp32_state(x, torch.full((300,), 0.5), torch.zeros(300), *_stbif_tensors(0.25, 3, -4))
    for got, want in zip(b, a[:4]):
        assert torch.equal(got, want)


# ------------------------------------------------------------------------------------------------
# EIF (functional/neuron.py:483-485): pins that do not retype the formula
# ------------------------------------------------------------------------------------------------
def test_eif_rheobase_fixed_point_and_lif_limit():
    """At v = theta_rh the exponential term is exactly delta_T, so x = v - v_rest - delta_T holds the potential
    still.  Far below theta_rh (in units of delta_T) the exponential vanishes and the neuron is a LIF with input decay
    resting at v_rest."""
    tau, dT, theta, v_rest = 2.0, 0.25, 0.5, -0.125  # dyadic: every intermediate value is exact
    v0 = torch.full((3,), theta)
    x = torch.full((1, 3), theta - v_rest - dT)
    _, _, h = no.multi_step("eif", x, v0, (tau, dT, theta, v_rest), True, 10.0, -1.0)
    assert torch.equal(h[0], v0)
    xs = seeded_randn((8, 200), 61, 0.0, 0.2, torch.float64)
    v0 = seeded_randn((200,), 62, 0.0, 0.1, torch.float64)
    p = (3.0, 0.01, 5.0, 0.1)  # theta_rh 490 delta_T above the potentials: exp() < 1e-200
    s_e, v_e, h_e = no.multi_step("eif", xs, v0, p, True, 1.0, -0.5)
    v = v0
    for t in range(8):
        h = v + (xs[t] - (v - 0.1)) / 3.0
        torch.testing.assert_close(h_e[t], h, rtol=1e-13, atol=1e-15)
        v = h  # no spikes at this drive
    assert float(s_e.sum()) == 0.0


@pytest.mark.parametrize("v_reset", [-0.1, None])
def test_eif_autograd_matches_finite_differences_of_the_smooth_network(v_reset):
    T, N, vth, alpha = 5, 6, 0.9, 2.0
    p = (2.5, 0.5, 0.6, 0.0)
    x = seeded_randn((T, N), 51, 0.4, 0.6, torch.float64)
    v0 = seeded_randn((N,), 52, 0.0, 0.3, torch.float64)
    gs = seeded_randn((T, N), 53, dtype=torch.float64)
    gv = seeded_randn((T, N), 54, dtype=torch.float64)
    smooth = no.surrogate("atan", alpha, spiking=False)

    def loss(x_, v0_):
        s, v, _ = no.multi_step("eif", x_, v0_, p, True, vth, v_reset, smooth)
        return float((s * gs).sum() + (v * gv).sum())

    ref = no.forward_backward("eif", x, v0, gs, gv, None, p, True, vth, v_reset, "atan", alpha, False, spiking=False)
    eps = 1e-6
    for (t, n) in [(0, 0), (2, 3), (T - 1, N - 1)]:
        xp, xm = x.clone(), x.clone()
        xp[t, n] += eps
        xm[t, n] -= eps
        assert (loss(xp, v0) - loss(xm, v0)) / (2 * eps) == pytest.approx(float(ref["grad_x"][t, n]), rel=1e-6, abs=1e-8)
    vp, vm = v0.clone(), v0.clone()
    vp[2] += eps
    vm[2] -= eps
    assert (loss(x, vp) - loss(x, vm)) / (2 * eps) == pytest.approx(float(ref["grad_v_init"][2]), rel=1e-6, abs=1e-8)


# ------------------------------------------------------------------------------------------------
# activation-aware IF (functional/neuron.py:577-584)
# ------------------------------------------------------------------------------------------------
def _aaif_by_hand(x_seq, threshold, offset, v_reset):
    """Plain Python floats, one neuron at a time; x_seq [T][n], threshold / offset one value per neuron."""
    T, n = len(x_seq), len(x_seq[0])
    v = [0.0 if v_reset is None else v_reset] * n
    spikes, volts = [], []
    for t in range(T):
        row_s, row_v = [], []
        for i in range(n):
            h = v[i] + x_seq[t][i]
            fired = 1.0 if h + offset[i] >= threshold[i] else 0.0
            v[i] = h - fired * threshold[i] if v_reset is None else (v_reset if fired else h)
            row_s.append(fired)
            row_v.append(v[i])
        spikes.append(row_s)
        volts.append(row_v)
    return spikes, volts


def test_activation_aware_if_on_the_reference_tests_literal_inputs():
    """Inputs of the reference's test_activation_aware_ifnode.py:253-352 against a neuron-by-neuron loop in Python
    floats (no value comes within 0.04 of a threshold, so fp32 and double agree on every spike)."""
    x = torch.tensor([[[0.8, 1.0], [1.2, 0.2]], [[0.6, 0.2], [0.4, 1.4]], [[0.3, 0.9], [0.1, 0.2]]])
    s, v = no.activation_aware_if_multi_step(x, torch.zeros(2, 2), 1.5, 0.25, -1, None)
    es, ev = _aaif_by_hand(x.flatten(1).tolist(), [1.5] * 4, [0.25] * 4, None)
    assert s.flatten(1).tolist() == es and float(s.sum()) > 0
    torch.testing.assert_close(v.flatten(1), torch.tensor(ev))

    x = torch.tensor([[[0.6, 1.0, 2.4], [1.1, 1.3, 1.0]], [[0.5, 0.4, 0.7], [0.2, 0.4, 1.3]]])
    th, off = [1.0, 1.5, 2.0], [0.0, 0.25, -0.25]
    s, v = no.activation_aware_if_multi_step(x, torch.zeros(2, 3), torch.tensor(th), torch.tensor(off), -1, None)
    es, ev = _aaif_by_hand(x.flatten(1).tolist(), th * 2, off * 2, None)
    assert s.flatten(1).tolist() == es and 0 < float(s.sum()) < s.numel()

    x = torch.tensor([[[1.1, 1.5]], [[0.2, 0.7]], [[0.8, 0.1]]])
    s, v = no.activation_aware_if_multi_step(x, torch.full((1, 2), 0.25), torch.tensor([1.0, 2.0]), 0.0, -1, 0.25)
    es, ev = _aaif_by_hand(x.flatten(1).tolist(), [1.0, 2.0], [0.0, 0.0], 0.25)
    assert s.flatten(1).tolist() == es
    torch.testing.assert_close(v.flatten(1), torch.tensor(ev))


def test_activation_aware_if_reduces_to_if():
    """Zero offset and a scalar threshold is the IF neuron, bit for bit; with a hard reset (where the threshold does
    not enter the reset) an offset o is the IF neuron with threshold theta - o on dyadic values; a 1-D parameter along
    channel_dim 0 of an [C, H, W] step treats every channel as its own scalar neuron."""
    x = seeded_randn((10, 3, 8, 8), 95, 0.3, 0.6)
    v0 = torch.zeros(3, 8, 8)
    for v_reset in (None, 0.0, -0.25):
        s, v = no.activation_aware_if_multi_step(x, v0 if v_reset is None else torch.full_like(v0, v_reset), 0.75, 0.0, 0, v_reset)
        es, ev, _ = no.multi_step("if", x, v0 if v_reset is None else torch.full_like(v0, v_reset), None, True, 0.75, v_reset)
        assert torch.equal(s, es) and torch.equal(v, ev)
    xd = torch.round(x * 64) / 64
    s, v = no.activation_aware_if_multi_step(xd, v0, 1.0, 0.25, 0, 0.0)
    es, ev, _ = no.multi_step("if", xd, v0, None, True, 0.75, 0.0)
    assert torch.equal(s, es) and torch.equal(v, ev)
    th = torch.tensor([0.5, 1.0, 1.5])
    s, v = no.activation_aware_if_multi_step(x, v0, th, 0.0, 0, None)
    for c in range(3):
        es, ev, _ = no.multi_step("if", x[:, c], v0[c], None, True, float(th[c]), None)
        assert torch.equal(s[:, c], es) and torch.equal(v[:, c], ev)


# ------------------------------------------------------------------------------------------------
# Izhikevich (functional/neuron.py:1514-1522)
# ------------------------------------------------------------------------------------------------
def test_izhikevich_reduces_to_qif_and_the_adaptation_current_decays_geometrically():
    """Without coupling (a = b = 0) and with w = 0 the membrane is the QIF neuron, bit for bit; a free adaptation
    current decays by (1 - 1/tau_w) per step; a spike adds b."""
    x = seeded_randn((10, 300), 111, 0.4, 0.5)
    v0 = seeded_randn((300,), 112, 0.0, 0.2)
    for v_reset in (0.0, -0.1):
        s, v, w, h = no.izhikevich_multi_step(x, v0, torch.zeros(300), (2.0, 1.0, -0.1, 0.8, 2.0, 0.0, 0.0), 1.0, v_reset)
        es, ev, eh = no.multi_step("qif", x, v0, (2.0, 1.0, -0.1, 0.8), True, 1.0, v_reset)
        assert torch.equal(s, es) and torch.equal(v, ev) and torch.equal(h, eh) and float(w.abs().max()) == 0.0
        assert 0.0 < float(s.mean()) < 0.9
    # x cancels the free current's pull on the membrane so that it never fires: w halves every step (tau_w = 2)
    w0 = torch.full((4,), 0.5)
    quiet = torch.zeros(6, 4)
    s, v, w, _ = no.izhikevich_multi_step(quiet, torch.full((4,), -0.1), w0, (2.0, 1.0, -0.1, 0.8, 2.0, 0.0, 0.0), 10.0, 0.0)
    assert float(s.sum()) == 0.0
    assert torch.equal(w[:, 0], torch.tensor([0.5 / 2 ** (t + 1) for t in range(6)]))
    # a spike adds b to w: drive one neuron over the threshold once
    x1 = torch.tensor([[3.0], [0.0]])
    s, v, w, _ = no.izhikevich_multi_step(x1, torch.zeros(1), torch.zeros(1), (2.0, 1.0, -0.1, 0.8, 2.0, 0.0, 0.25), 1.0, 0.0)
    assert s.flatten().tolist() == [1.0, 0.0] and float(w[0]) == 0.25 and float(w[1]) == 0.125


GRID_IZH = [(vr, det, sg) for vr in (0.0, -0.2, None) for det in (False, True) for sg in ("atan", "sigmoid")]


@pytest.mark.parametrize("v_reset,detach,sg", GRID_IZH)
def test_izhikevich_recurrence_equals_autograd_float64(v_reset, detach, sg):
    T, N, vth = 6, 129, 0.8
    alpha = no.SG_DEFAULT_ALPHA[sg]
    params = (2.5, 0.7, -0.1, 0.6, 3.0, 0.3, 0.2)
    scale = 0.5 if v_reset is not None else 0.25
    x = seeded_randn((T, N), 121, 0.3, scale, torch.float64).requires_grad_()
    v0 = seeded_randn((N,), 122, 0.0, 0.2, torch.float64).requires_grad_()
    w0 = seeded_randn((N,), 123, 0.0, 0.2, torch.float64).requires_grad_()
    gs, gv, gw = (seeded_randn((T, N), 124 + i, 0.0, 1.0 if i == 0 else 0.2, torch.float64) for i in range(3))
    gvl, gwl = seeded_randn((N,), 128, dtype=torch.float64), seeded_randn((N,), 129, dtype=torch.float64)
    s, v, w, h = no.izhikevich_multi_step(x, v0, w0, params, vth, v_reset, no.surrogate(sg, alpha), detach)
    assert bool(torch.isfinite(v).all())
    torch.autograd.backward([s, v, w, v[-1], w[-1]], [gs, gv, gw, gvl, gwl])
    gx, gv0, gw0 = bptt_oracle.bptt_izhikevich(h.detach().numpy(), v0.detach().numpy(), _np_sg_prime(sg, alpha), gs.numpy(),
                                               gv.numpy(), gw.numpy(), gvl.numpy(), gwl.numpy(), params, vth, v_reset, detach)
    np.testing.assert_allclose(gx, x.grad.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(gv0, v0.grad.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(gw0, w0.grad.numpy(), rtol=1e-10, atol=1e-12)


def test_izhikevich_autograd_matches_finite_differences_of_the_smooth_network():
    T, N, vth, alpha = 5, 4, 0.9, 2.0
    params = (2.5, 0.7, -0.1, 0.6, 3.0, 0.3, 0.2)
    x = seeded_randn((T, N), 131, 0.3, 0.4, torch.float64)
    v0 = seeded_randn((N,), 132, 0.0, 0.2, torch.float64)
    w0 = seeded_randn((N,), 133, 0.0, 0.2, torch.float64)
    gs, gv, gw = (seeded_randn((T, N), 134 + i, dtype=torch.float64) for i in range(3))
    smooth = no.surrogate("atan", alpha, spiking=False)

    def loss(x_, v_, w_):
        s, v, w, _ = no.izhikevich_multi_step(x_, v_, w_, params, vth, -0.1, smooth)
        return (s * gs).sum() + (v * gv).sum() + (w * gw).sum()

    xa, va, wa = x.clone().requires_grad_(), v0.clone().requires_grad_(), w0.clone().requires_grad_()
    loss(xa, va, wa).backward()
    eps = 1e-6
    for (t, n) in [(0, 0), (2, 3), (T - 1, 1)]:
        xp, xm = x.clone(), x.clone()
        xp[t, n] += eps
        xm[t, n] -= eps
        assert float(loss(xp, v0, w0) - loss(xm, v0, w0)) / (2 * eps) == pytest.approx(float(xa.grad[t, n]), rel=1e-6, abs=1e-8)
    wp, wm = w0.clone(), w0.clone()
    wp[2] += eps
    wm[2] -= eps
    assert float(loss(x, v0, wp) - loss(x, v0, wm)) / (2 * eps) == pytest.approx(float(wa.grad[2]), rel=1e-6, abs=1e-8)


# ------------------------------------------------------------------------------------------------
# 8-bit floating-point storage: the conversion the expected values rely on, and the recipe's structure
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("storage", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_torch_float8_conversion_is_round_to_nearest_even_over_the_code_table(storage):
    """Brute force: the nearest of the 256 decoded codes, ties to the code with an even mantissa; beyond the largest
    finite value e4m3fn (no infinity) gives NaN once the value rounds past it, e5m2 gives infinity."""
    codes = torch.arange(256, dtype=torch.uint8)
    table = codes.view(storage).float().double()
    finite = torch.isfinite(table)
    pos = [(float(table[i]), int(codes[i])) for i in range(256) if finite[i] and int(codes[i]) < 128]
    pos.sort()
    top, step = pos[-1][0], pos[-1][0] - pos[-2][0]
    rng = np.random.default_rng(5)
    samples = np.concatenate([rng.normal(0, 1, 4000), rng.normal(0, 2 ** -7, 2000), rng.normal(0, 100, 2000),
                              [(a[0] + b[0]) / 2 for a, b in zip(pos[:-1], pos[1:])], [top + step / 2, top + step * 0.51, top * 3]])
    samples = samples.astype(np.float32)
    got = torch.from_numpy(samples).to(storage).view(torch.uint8).numpy()
    for x, code in zip(samples.astype(np.float64), got):
        mag = abs(x)
        # the tie between the largest finite value and the first value past it goes to whichever code is even:
        # e4m3fn's largest finite code (0x7e) is even and keeps it, e5m2's (0x7b) is odd and loses it to infinity
        top_is_even = (pos[-1][1] & 1) == 0
        want_special = mag > top + step / 2 or (mag == top + step / 2 and not top_is_even)
        if want_special:
            decoded = float(torch.tensor([code], dtype=torch.uint8).view(storage).float())
            assert math.isnan(decoded) if storage == torch.float8_e4m3fn else math.isinf(decoded), (x, code)
            continue
        best = min(pos, key=lambda vc: (abs(vc[0] - mag), vc[1] & 1))  # nearest; on a tie the even code
        assert (code & 0x7f) == best[1], (x, code, best)
        assert (code >> 7) == (1 if np.signbit(x) else 0)


@pytest.mark.parametrize("storage", [torch.float8_e4m3fn, torch.float8_e5m2, torch.bfloat16])
@pytest.mark.parametrize("kind,k", [("if", 0.0), ("lif", 0.5), ("plif", 0.25)])
@pytest.mark.parametrize("v_reset", [0.0, -0.25, None])
def test_mixed_precision_recipe_is_the_fp32_recurrence_on_rounded_inputs(storage, kind, k, v_reset):
    """Structure of the recipe: inputs rounded to the storage dtype, the fp32 recurrence (the oracle pinned above) on
    them with the state never rounded, stored values rounded once.  Rounding what is stored cannot change a spike."""
    q = lambda t: t.to(storage).float()
    x, v0 = seeded_randn((9, 300), 61, 0.6, 0.9), seeded_randn((300,), 62, 0.0, 0.3)
    s, v, h, raw = no.multi_step_mixed_precision(kind, x, v0, storage, k=k, v_reset=v_reset, return_raw_h=True)
    p = {"if": None, "lif": 1.0 / k if k else None, "plif": torch.tensor(math.log(k / (1 - k))) if k else None}[kind]
    es, ev, eh = no.multi_step(kind, q(x), q(v0), p, True, 1.0, v_reset)
    assert torch.equal(s, es) and torch.equal(raw, eh)
    assert torch.equal(h, q(eh)) and torch.equal(v, q(ev)) and 0.005 < float(s.mean()) < 0.9
