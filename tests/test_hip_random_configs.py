"""Seeded random sweep over the drop-in boundary: a hip node against the torch node on the CPU.

Each case draws the neuron, its parameters, the shape (ragged sizes included), the surrogate, the reset mode,
store_v_seq, the backward path and a second call that continues from the carried state.  fp32: spikes and
states bit-exact, gradients to 1e-5; fp16 / bf16 in every-op-rounded mode (IF, LIF, QIF, ILIF): spikes and states
bit-exact, gradients to a few 16-bit ulps of the largest gradient (the torch node rounds every backward op).
"""

import numpy as np
import pytest
import torch

from spikingjelly_amd import configure
from spikingjelly_amd.activation_based import functional, neuron, surrogate

from helpers import bits_equal

pytestmark = pytest.mark.gpu

SURROGATES = [surrogate.ATan, surrogate.Sigmoid, surrogate.PiecewiseQuadratic, surrogate.PiecewiseExp,
              surrogate.SoftSign, surrogate.SuperSpike, surrogate.Erf]


def _draw(seed):
    rng = np.random.default_rng(seed)
    kind = rng.choice(["if", "lif", "plif", "qif"])
    dtype = rng.choice([torch.float32, torch.float32, torch.float16, torch.bfloat16])
    if kind == "plif" and dtype != torch.float32:
        dtype = torch.float32  # 16-bit PLIF rounds k on the device; covered at operator level with a shared k
    T = int(rng.choice([1, 2, 3, 5, 8, 16, 33, 48]))
    shape = tuple(int(v) for v in rng.choice([1, 2, 3, 4, 7, 8, 12, 32, 37, 64, 100], size=int(rng.integers(1, 4))))
    v_reset = [0.0, -0.25, None][int(rng.integers(0, 3))]
    kw = dict(v_threshold=float(rng.choice([0.5, 1.0, 1.25])), v_reset=v_reset, detach_reset=bool(rng.integers(0, 2)),
              surrogate_function=SURROGATES[int(rng.integers(0, len(SURROGATES)))](), store_v_seq=bool(rng.integers(0, 2)))
    if kind == "lif":
        cls, extra = neuron.LIFNode, dict(tau=float(rng.choice([2.0, 3.0, 1.5, 10.0])), decay_input=bool(rng.integers(0, 2)))
    elif kind == "plif":
        cls, extra = neuron.ParametricLIFNode, dict(init_tau=2.0, decay_input=bool(rng.integers(0, 2)))
    elif kind == "qif":
        cls, extra = neuron.QIFNode, dict(tau=float(rng.choice([2.0, 3.0])), v_c=0.5, a0=float(rng.choice([0.5, 1.0])), v_rest=0.0)
        kw["v_threshold"] = 1.0
        kw["v_reset"] = [0.0, -0.25][int(rng.integers(0, 2))]  # a soft reset lets the quadratic term diverge
    else:
        cls, extra = neuron.IFNode, {}
    kw.update(extra)
    recompute = bool(rng.integers(0, 2))
    scale = 0.4 if kind == "qif" else 1.0
    return kind, cls, kw, dtype, T, shape, recompute, scale, int(rng.integers(0, 1 << 30))


def _draw_ilif(seed):
    """The integer-valued LIF: time constant, threshold (a power of two or not), count limit, gradient window."""
    rng = np.random.default_rng(10_000 + seed)
    dtype = rng.choice([torch.float32, torch.float32, torch.float16, torch.bfloat16])
    T = int(rng.choice([1, 2, 3, 5, 8, 16, 33, 48]))
    shape = tuple(int(v) for v in rng.choice([1, 2, 3, 4, 7, 8, 12, 32, 37, 64, 100], size=int(rng.integers(1, 4))))
    levels = int(rng.choice([1, 2, 4, 7]))
    window = [None, (-0.5, levels + 0.5), (0.25, levels - 0.25)][int(rng.integers(0, 3))]
    v_th = float(rng.choice([0.5, 1.0, 0.7, 1.25]))
    kw = dict(tau=float(rng.choice([4.0 / 3.0, 2.0, 1.6, 10.0])), v_threshold=v_th,
              surrogate_function=surrogate.MultiLevelSpikeCount(levels, grad_window=window),
              detach_reset=bool(rng.integers(0, 2)), store_v_seq=bool(rng.integers(0, 2)))
    # drive the neuron over its whole range of counts
    return "ilif", neuron.ILIFNode, kw, dtype, T, shape, bool(rng.integers(0, 2)), v_th * levels * 0.6, int(rng.integers(0, 1 << 30))


def _draw_izhikevich(seed):
    """Two coupled states: both time constants (exact reciprocals or not), the coupling, hard reset (a soft reset lets
    the quadratic term diverge on a random drive), saved-h or replaying backward."""
    rng = np.random.default_rng(20_000 + seed)
    dtype = rng.choice([torch.float32, torch.float32, torch.float32, torch.float16, torch.bfloat16])
    T = int(rng.choice([1, 2, 3, 5, 8, 16, 33]))
    shape = tuple(int(v) for v in rng.choice([1, 2, 3, 4, 7, 8, 12, 32, 37, 64, 100], size=int(rng.integers(1, 4))))
    kw = dict(tau=float(rng.choice([2.0, 2.5, 4.0, 10.0])), tau_w=float(rng.choice([2.0, 3.0, 8.0])), v_c=float(rng.choice([0.5, 0.8])),
              a0=float(rng.choice([0.5, 1.0])), v_rest=float(rng.choice([0.0, -0.1])), w_rest=float(rng.choice([0.0, 0.05])),
              a=float(rng.choice([0.0, 0.3, -0.2])), b=float(rng.choice([0.0, 0.2])), v_threshold=1.0,
              v_reset=float(rng.choice([0.0, -0.25])), detach_reset=bool(rng.integers(0, 2)),
              surrogate_function=SURROGATES[int(rng.integers(0, len(SURROGATES)))](), store_v_seq=bool(rng.integers(0, 2)))
    return "izhikevich", neuron.IzhikevichNode, kw, dtype, T, shape, bool(rng.integers(0, 2)), 0.5, int(rng.integers(0, 1 << 30))


@pytest.mark.parametrize("seed", range(80))
def test_random_izhikevich_configuration(seed):
    _run_case(*_draw_izhikevich(seed))


@pytest.mark.parametrize("seed", range(300))
def test_random_configuration(seed):
    _run_case(*_draw(seed))


@pytest.mark.parametrize("seed", range(100))
def test_random_ilif_configuration(seed):
    _run_case(*_draw_ilif(seed))


def _run_case(kind, cls, kw, dtype, T, shape, recompute, scale, data_seed):
    g = torch.Generator().manual_seed(data_seed)
    x = (torch.randn((T,) + shape, generator=g) * scale + 0.4).to(dtype)
    x2 = (torch.randn((T,) + shape, generator=g) * scale + 0.4).to(dtype)
    gs = torch.randn((T,) + shape, generator=g).to(dtype)
    old = (configure.hip_backward_recompute, configure.hip_half_precision_mode)
    configure.hip_backward_recompute, configure.hip_half_precision_mode = recompute, "torch"
    try:
        a = cls(step_mode="m", backend="torch", **kw)
        b = cls(step_mode="m", backend="hip", **kw).cuda()
        xa, xb = x.clone().requires_grad_(), x.cuda().requires_grad_()
        sa, sb = a(xa), b(xb)
        assert bits_equal(sb.cpu(), sa.detach()), "spikes"
        assert bits_equal(b.v.detach().cpu(), a.v.detach()), "state"
        if kind == "izhikevich":
            assert bits_equal(b.w.detach().cpu(), a.w.detach()), "adaptation state"
        if kw["store_v_seq"]:
            assert bits_equal(b.v_seq.detach().cpu(), a.v_seq.detach()), "v_seq"
        la = (sa.float() * gs.float()).sum() + 0.5 * a.v.float().sum()
        lb = (sb.float() * gs.cuda().float()).sum() + 0.5 * b.v.float().sum()
        la.backward()
        lb.backward()
        if dtype == torch.float32:
            torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=1e-5, atol=2e-6)
        else:
            # the torch node back-propagates in 16-bit arithmetic, rounding every op over T steps; the kernel keeps
            # fp32 and rounds once, so single elements differ by a few 16-bit ulps of the largest gradient
            got, want = xb.grad.float().cpu(), xa.grad.float()
            assert float((got - want).abs().max()) <= 3e-2 * float(want.abs().max()) + 1e-3
        if kind == "plif":
            torch.testing.assert_close(b.w.grad.cpu(), a.w.grad, rtol=1e-4, atol=1e-5)
        # second call: the state is now an ordinary tensor carried over from the first call
        sa2, sb2 = a(x2), b(x2.cuda())
        assert bits_equal(sb2.cpu(), sa2.detach()), "spikes of the second call"
        assert bits_equal(b.v.detach().cpu(), a.v.detach()), "state after the second call"
        if kind == "izhikevich":
            assert bits_equal(b.w.detach().cpu(), a.w.detach()), "adaptation state after the second call"
    finally:
        configure.hip_backward_recompute, configure.hip_half_precision_mode = old
        functional.reset_net(a)
        functional.reset_net(b)
