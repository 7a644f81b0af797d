"""ST-BIF (SpikeZIP's signed ternary neuron) on the hip backend against the oracle and the torch backend.

Inference only.  Bars: outputs and all three states bit-exact against the torch backend's step (fp32, and fp16 / bf16
with every op rounded), bit-exact against the Triton kernel's arithmetic in the fp32-state mode, and the released
total equal to the quantiser the neuron stands for.
"""

import pytest
import torch

from oracle import stbif_oracle
from spikingjelly_amd import configure
from spikingjelly_amd.activation_based import functional, neuron

from helpers import bits_equal, require_device_memory, seeded_randn

pytestmark = pytest.mark.gpu


def _scalars(scale, pos_max, neg_min):
    return torch.tensor(float(scale)), torch.tensor(float(pos_max)), torch.tensor(float(neg_min))


def _states(n, dtype, seed=None):
    if seed is None:
        return torch.full((n,), 0.5, dtype=dtype), torch.zeros(n, dtype=dtype)
    # a carried state: a residual anywhere in [0, 1) and an integer inside the bounds
    g = torch.Generator().manual_seed(seed)
    return torch.rand(n, generator=g).to(dtype), torch.randint(-2, 3, (n,), generator=g).to(dtype)


@pytest.mark.parametrize("scale,pos_max,neg_min", [(0.25, 3, -4), (0.125, 7, 0), (0.3, 1, -2)])
@pytest.mark.parametrize("T,N", [(16, 4096), (7, 111), (33, 260), (1, 4)])
@pytest.mark.parametrize("carried", [False, True])
def test_fp32_bit_exact_against_the_torch_step(scale, pos_max, neg_min, T, N, carried):
    x = seeded_randn((T, N), 100 + T, 0.05, 0.4)
    x[T // 2] = 0.0  # a silent step in the middle
    q0, a0 = _states(N, torch.float32, 7 if carried else None)
    th = _scalars(scale, pos_max, neg_min)
    eo, eq, ea, ec, ework = stbif_oracle.multi_step(x, q0, a0, *th)
    out, q, acc, cur, work = functional.stbif_multi_step_hip(x.cuda(), q0.cuda(), a0.cuda(), *[t.cuda() for t in th])
    assert bits_equal(out.cpu(), eo) and bits_equal(q.cpu(), eq) and bits_equal(acc.cpu(), ea) and bits_equal(cur.cpu(), ec)
    assert bool(work.item()) is ework
    if T * N > 1000:
        assert set(torch.unique(ec).tolist()) <= {-1.0, 0.0, 1.0} and float(eo.abs().max()) > 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,N", [(12, 2048), (5, 77)])
@pytest.mark.parametrize("scale,pos_max,neg_min", [(0.25, 3, -4), (0.3, 7, -8)])
def test_16bit_both_modes(dtype, T, N, scale, pos_max, neg_min):
    x = seeded_randn((T, N), 21, 0.05, 0.4).to(dtype)
    q0, a0 = _states(N, dtype)
    th = _scalars(scale, pos_max, neg_min)
    old = configure.hip_half_precision_mode
    try:
        configure.hip_half_precision_mode = "torch"
        eo, eq, ea, ec, _ = stbif_oracle.multi_step(x, q0, a0, *th)
        got = functional.stbif_multi_step_hip(x.cuda(), q0.cuda(), a0.cuda(), *[t.cuda() for t in th])
        for g, e in zip(got[:4], (eo, eq, ea, ec)):
            assert bits_equal(g.cpu(), e)
        configure.hip_half_precision_mode = "fp32_state"
        want = stbif_oracle.multi_step_fp32_state(x, q0, a0, *th)
        got = functional.stbif_multi_step_hip(x.cuda(), q0.cuda(), a0.cuda(), *[t.cuda() for t in th])
        for g, e in zip(got[:4], want):
            assert bits_equal(g.cpu(), e)
    finally:
        configure.hip_half_precision_mode = old


def test_reference_literal_cases_through_the_hip_backend():
    """Inputs and expectations of the reference's test_ann2snn_transformer.py:792-803, 975-1010 and
    test_functional_neuron.py:690-705."""
    node = neuron.STBIFNeuron(0.25, level=8, sym=True).cuda()
    node.backend = "hip"
    x = torch.tensor([[-0.75, -0.2, 0.3, 0.9]]).cuda()
    total = None
    for step in range(16):
        out = node(x if step == 0 else torch.zeros_like(x))
        total = out if total is None else total + out
    assert total.cpu().tolist() == [[-0.75, -0.25, 0.25, 0.75]]
    assert set(torch.unique(node.cur_output).tolist()) <= {-1.0, 0.0, 1.0}
    torch.testing.assert_close(node.accumulated, total)

    zeros = torch.zeros(6, device="cuda")
    acc = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, -2.5], device="cuda")
    th = [t.cuda() for t in _scalars(0.1, 10, -10)]
    out, q, acc2, cur, work = functional.stbif_single_step_hip(zeros, torch.full_like(zeros, 0.5), acc, *th)
    assert torch.equal(acc2.cpu(), torch.tensor([0.0, 2.0, 2.0, 0.0, -2.0, -2.0]))
    assert bits_equal(acc2.cpu(), stbif_oracle.step(zeros.cpu(), torch.full((6,), 0.5), acc.cpu(), *_scalars(0.1, 10, -10))[2])
    assert not bool(work.item()) and float(out.abs().max()) == 0.0

    node = neuron.STBIFNeuron(0.25, level=8, sym=True).cuda()
    node.backend = "hip"
    z = torch.zeros(2, 3, device="cuda")
    node(z)
    assert not node.is_work
    node(torch.full_like(z, 0.25))
    assert node.is_work
    node.reset()
    node.step_mode = "m"
    node(torch.stack([z, z]))
    assert not node.is_work
    node(torch.stack([z, torch.full_like(z, 0.25)]))
    assert node.is_work


@pytest.mark.parametrize("sym", [True, False])
def test_hip_node_matches_torch_node_and_the_quantiser(sym):
    level, scale = 16, 0.125
    a = neuron.STBIFNeuron(scale, level=level, sym=sym, step_mode="m")
    b = neuron.STBIFNeuron(scale, level=level, sym=sym, step_mode="m").cuda()
    b.backend = "hip"
    x = seeded_randn((1, 8, 33), 5, 0.2, 0.8)
    x_seq = torch.cat([x, torch.zeros(31, 8, 33)])
    ya, yb = a(x_seq), b(x_seq.cuda())
    assert bits_equal(yb.cpu(), ya) and a.is_work == b.is_work
    for name in ("q", "acc_q", "cur_output"):
        assert bits_equal(getattr(b, name).cpu(), getattr(a, name)), name
    lo, hi = (-level // 2, level // 2 - 1) if sym else (0, level - 1)
    torch.testing.assert_close(yb.sum(0).cpu(), torch.clamp(torch.floor(x[0] / scale + 0.5), lo, hi) * scale)
    # a second call continues from the carried states
    x2 = seeded_randn((4, 8, 33), 6, 0.0, 0.3)
    assert bits_equal(b(x2.cuda()).cpu(), a(x2))
    # single-step mode on the same states
    functional.set_step_mode(a, "s")
    functional.set_step_mode(b, "s")
    assert bits_equal(b(x2[0].cuda()).cpu(), a(x2[0]))
    functional.reset_net(a)
    functional.reset_net(b)
    assert b.q is None and b.is_work is False


def test_full_size_against_the_quantiser():
    """T = 16 over 33.5 M neurons: the released total of every neuron equals the quantiser of its input, and column
    blocks equal the torch step bit for bit."""
    require_device_memory(12)
    T, N, scale = 16, 256 * 128 * 32 * 32, 0.25
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.zeros((T, N), device="cuda")
    x[0] = torch.randn(N, generator=g, device="cuda") * 0.6
    x[1] = torch.randn(N, generator=g, device="cuda") * 0.1
    th = [t.cuda() for t in _scalars(scale, 3, -4)]
    q0 = torch.full((1,), 0.5, device="cuda").expand(N)
    a0 = torch.zeros((1,), device="cuda").expand(N)
    out, q, acc, cur, work = functional.stbif_multi_step_hip(x, q0, a0, *th)
    total = x[0].double() + x[1].double()
    want = torch.clamp(torch.floor(total / scale + 0.5), -4, 3)
    # the two inputs arrive one step apart, so a unit released after the first may be taken back after the second:
    # the released integer still ends at the quantiser of the total.  The neuron adds in fp32, so an input within
    # rounding distance of a quantisation boundary may land on the other side of it.
    near_boundary = ((total / scale + 0.5) - torch.round(total / scale + 0.5)).abs() < 1e-5
    assert bool(((acc.double() == want) | near_boundary).all()) and bool(work.item())
    assert float((acc.double() - want).abs().max()) <= 1.0
    assert torch.equal(out.sum(0), acc * scale)
    cols = torch.arange(0, 4096, device="cuda") + (N // 3)
    eo, eq, ea, ec, _ = stbif_oracle.multi_step(x[:, cols].cpu(), torch.full((4096,), 0.5), torch.zeros(4096),
                                                *_scalars(scale, 3, -4))
    assert bits_equal(out[:, cols].cpu(), eo) and bits_equal(q[cols].cpu(), eq) and bits_equal(cur[cols].cpu(), ec)
