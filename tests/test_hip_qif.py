"""Quadratic integrate-and-fire neuron on the hip backend against the oracle and the torch backend.

Bars as for IF / LIF / PLIF: spikes, h, v bit-exact in fp32 and in every-op-rounded 16-bit mode; gradients
within rtol 1e-5 (fp32) / 1e-2 (16-bit) of autograd through the oracle.
"""

import pytest
import torch

from oracle import neuron_oracle as no
from spikingjelly_amd import configure
from spikingjelly_amd.activation_based import functional, neuron, surrogate

from helpers import bits_equal, seeded_randn

pytestmark = pytest.mark.gpu

GRAD_RTOL, GRAD_ATOL = 1e-5, 1e-6


@pytest.fixture(scope="module")
def K():
    from spikingjelly_amd.activation_based.hip_kernel import library, neuron_kernel

    library.load()
    return neuron_kernel


PARAMS = [  # tau, a0, v_rest, v_c
    (2.0, 1.0, 0.0, 0.8),
    (3.0, 0.7, -0.05, 0.6),
    (10.0, 1.5, 0.1, 0.5),
]


@pytest.mark.parametrize("tau,a0,v_rest,v_c", PARAMS)
@pytest.mark.parametrize("v_reset", [-0.1, 0.0, None])
@pytest.mark.parametrize("T,N,recompute", [(16, 4096, False), (16, 4096, True), (7, 111, False), (33, 260, False),
                                           (33, 260, True), (1, 4, False), (1, 4, True)])  # replay: N % 4 == 0
def test_forward_bit_exact_and_gradients_fp32(K, tau, a0, v_rest, v_c, v_reset, T, N, recompute):
    # with a soft reset the quadratic term escapes to infinity once v exceeds about 2: keep the drive small there
    x = seeded_randn((T, N), 100 + T, 0.5, 1.0) if v_reset is not None else seeded_randn((T, N), 100 + T, 0.3, 0.4)
    v0 = seeded_randn((N,), 200 + N, 0.0, 0.3)
    gs, gv = seeded_randn((T, N), 300 + T), seeded_randn((T, N), 400 + T, 0.0, 0.1)
    vth = 1.0
    ref = no.forward_backward("qif", x, v0, gs, gv, None, (tau, a0, v_rest, v_c), True, vth, v_reset, "atan", 2.0, False)
    assert bool(torch.isfinite(ref["v_seq"]).all()) and bool(torch.isfinite(ref["grad_x"]).all())
    if T * N > 1000:
        assert 0.0 < float(ref["spike_seq"].mean()) < 0.9
    soft = v_reset is None
    xd = x.cuda().requires_grad_()
    vd = v0.cuda().requires_grad_()
    s, v_seq, v_last, h = K.hip_multistep_qif_forward(xd, vd, vth, 0.0 if soft else v_reset, soft, False, tau, v_rest, v_c,
                                                      a0, 1, 2.0, True, 0, recompute)
    assert bits_equal(s.cpu(), ref["spike_seq"])
    assert bits_equal(v_seq.cpu(), ref["v_seq"])
    assert bits_equal(v_last.cpu(), ref["v_seq"][-1])
    if not recompute:
        assert bits_equal(h.cpu(), ref["h_seq"])
    torch.autograd.backward([s, v_seq], [gs.cuda(), gv.cuda()])
    torch.testing.assert_close(xd.grad.cpu(), ref["grad_x"], rtol=GRAD_RTOL, atol=GRAD_ATOL)
    torch.testing.assert_close(vd.grad.cpu(), ref["grad_v_init"], rtol=GRAD_RTOL, atol=GRAD_ATOL)


@pytest.mark.parametrize("detach_reset", [False, True])
@pytest.mark.parametrize("sg_name,sg_id,alpha", [("sigmoid", 0, 4.0), ("atan", 1, 2.0)])
def test_grad_v_last_and_detach_reset(K, detach_reset, sg_name, sg_id, alpha):
    """store_v_seq=False: only the gradient of the last state enters (unscaled by dh/dv)."""
    T, N = 9, 256
    p = (2.0, 1.0, 0.0, 0.8)
    x = seeded_randn((T, N), 7, 0.5, 1.0)
    v0 = seeded_randn((N,), 8, 0.0, 0.3)
    gs, gl = seeded_randn((T, N), 9), seeded_randn((N,), 10)
    ref = no.forward_backward("qif", x, v0, gs, None, gl, p, True, 1.0, -0.1, sg_name, alpha, detach_reset)
    for recompute in (False, True):
        xd, vd = x.cuda().requires_grad_(), v0.cuda().requires_grad_()
        s, _, v_last, _ = K.hip_multistep_qif_forward(xd, vd, 1.0, -0.1, False, detach_reset, p[0], p[2], p[3], p[1], sg_id,
                                                      alpha, False, 0, recompute)
        torch.autograd.backward([s, v_last], [gs.cuda(), gl.cuda()])
        torch.testing.assert_close(xd.grad.cpu(), ref["grad_x"], rtol=GRAD_RTOL, atol=GRAD_ATOL)
        torch.testing.assert_close(vd.grad.cpu(), ref["grad_v_init"], rtol=GRAD_RTOL, atol=GRAD_ATOL)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,N", [(8, 2048), (5, 77)])
def test_every_op_rounded_16bit_equals_torch_ops_on_half_tensors(K, dtype, T, N):
    """The torch backend on half tensors rounds after every op (a Python scalar is rounded to the tensor dtype for
    add / sub, kept in fp32 for mul / div): spikes, h and v must match it bit for bit."""
    p = (3.0, 0.7, -0.05, 0.6)
    x = seeded_randn((T, N), 21, 0.5, 1.0).to(dtype)
    v0 = seeded_randn((N,), 22, 0.0, 0.3).to(dtype)
    es, ev, eh = no.multi_step("qif", x, v0, p, True, 1.0, -0.1)
    s, v_seq, v_last, h = K.hip_multistep_qif_forward(x.cuda(), v0.cuda(), 1.0, -0.1, False, False, p[0], p[2], p[3], p[1],
                                                      1, 2.0, True, 0, False)
    assert bits_equal(s.cpu(), es) and bits_equal(h.cpu(), eh) and bits_equal(v_seq.cpu(), ev)


@pytest.mark.parametrize("v_reset", [-0.1, None])
@pytest.mark.parametrize("store_v_seq", [False, True])
def test_hip_node_matches_torch_node(v_reset, store_v_seq):
    kw = dict(tau=2.0, v_c=0.8, a0=1.0, v_threshold=1.0, v_rest=0.0, v_reset=v_reset,
              surrogate_function=surrogate.ATan(), store_v_seq=store_v_seq)
    a = neuron.QIFNode(step_mode="m", backend="torch", **kw)
    b = neuron.QIFNode(step_mode="m", backend="hip", **kw).cuda()
    x = seeded_randn((6, 4, 12, 4), 20260428, 0.3, 0.4)
    xa, xb = x.clone().requires_grad_(), x.cuda().requires_grad_()
    sa, sb = a(xa), b(xb)
    (sa.sum() + 0.5 * a.v.sum()).backward()
    (sb.sum() + 0.5 * b.v.sum()).backward()
    assert 0.0 < float(sa.detach().mean()) < 0.9
    assert bits_equal(sb.cpu(), sa.detach())
    assert bits_equal(b.v.detach().cpu(), a.v.detach())
    if store_v_seq:
        assert bits_equal(b.v_seq.detach().cpu(), a.v_seq.detach())
    torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=GRAD_RTOL, atol=GRAD_ATOL)
    # a second call continues from the carried state (an ordinary tensor now, with its own gradient path)
    sa2, sb2 = a(xa.detach()), b(xb.detach())
    assert bits_equal(sb2.cpu(), sa2.detach())
    functional.reset_net(a)
    functional.reset_net(b)


def test_module_rejects_what_the_reference_rejects():
    with pytest.raises(AssertionError):
        neuron.QIFNode(tau=1.0)
    with pytest.raises(AssertionError):
        neuron.QIFNode(a0=0.0)
    node = neuron.QIFNode()
    assert node.supported_backends == ("torch",)
    node.step_mode = "m"
    assert node.supported_backends == ("torch", "hip")
    assert "v_c=0.8" in repr(node) and "a0=1.0" in repr(node)
