"""Integer-valued LIF (ILIF) on the hip backend against the oracle and the torch backend.

Bars as for the binary neurons: counts, h and v bit-exact in fp32 and in every-op-rounded 16-bit mode; gradients
within rtol 1e-5 (fp32) / 1e-2 (16-bit) of autograd through the oracle.  The gradient window is a hard mask on
h / v_th, so bit-exact h is also what makes the masks of the two sides agree.
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


PARAMS = [  # tau, v_th, levels, gradient window
    (4.0 / 3.0, 1.0, 4, (0.0, 4.0)),
    (2.0, 0.5, 2, (-0.5, 2.25)),
    (1.6, 0.7, 7, (0.0, 7.0)),
]


@pytest.mark.parametrize("tau,v_th,levels,window", PARAMS)
@pytest.mark.parametrize("T,N,recompute", [(16, 4096, False), (16, 4096, True), (7, 111, False), (33, 260, False),
                                           (33, 260, True), (1, 4, False), (1, 4, True)])  # replay: N % 4 == 0
@pytest.mark.parametrize("detach", [False, True])
def test_forward_bit_exact_and_gradients_fp32(K, tau, v_th, levels, window, T, N, recompute, detach):
    x = seeded_randn((T, N), 100 + T, 0.6 * v_th * levels / 2, v_th * levels / 2)
    v0 = seeded_randn((N,), 200 + N, 0.0, 0.3)
    gs, gv = seeded_randn((T, N), 300 + T), seeded_randn((T, N), 400 + T, 0.0, 0.1)
    ref = no.forward_backward("ilif", x, v0, gs, gv, None, tau, False, v_th, None, detach_reset=detach,
                              sg=no.multi_level_spike_count(levels, window))
    if T * N > 1000:
        assert float(ref["spike_seq"].max()) == levels and float(ref["spike_seq"].min()) == 0.0
        z = ref["h_seq"] / v_th
        assert 0.05 < float(((z >= window[0]) & (z <= window[1])).float().mean()) < 0.95
    xd = x.cuda().requires_grad_()
    vd = v0.cuda().requires_grad_()
    s, v_seq, v_last, h = K.hip_multistep_ilif_forward(xd, vd, tau, v_th, levels, window[0], window[1], detach, True, 0,
                                                       recompute)
    assert bits_equal(s.cpu(), ref["spike_seq"])
    assert bits_equal(v_seq.cpu(), ref["v_seq"])
    assert bits_equal(v_last.cpu(), ref["v_seq"][-1])
    if not recompute:
        assert bits_equal(h.cpu(), ref["h_seq"])
    torch.autograd.backward([s, v_seq], [gs.cuda(), gv.cuda()])
    torch.testing.assert_close(xd.grad.cpu(), ref["grad_x"], rtol=GRAD_RTOL, atol=GRAD_ATOL)
    torch.testing.assert_close(vd.grad.cpu(), ref["grad_v_init"], rtol=GRAD_RTOL, atol=GRAD_ATOL)


@pytest.mark.parametrize("recompute", [False, True])
def test_grad_v_last_without_v_seq_and_inference_op(K, recompute):
    T, N = 9, 256
    tau, v_th, levels = 1.6, 0.7, 3
    x = seeded_randn((T, N), 7, 0.8, 1.0)
    v0 = seeded_randn((N,), 8, 0.0, 0.3)
    gs, gl = seeded_randn((T, N), 9), seeded_randn((N,), 10)
    ref = no.forward_backward("ilif", x, v0, gs, None, gl, tau, False, v_th, None, sg=no.multi_level_spike_count(levels))
    xd, vd = x.cuda().requires_grad_(), v0.cuda().requires_grad_()
    s, v_seq, v_last, _ = K.hip_multistep_ilif_forward(xd, vd, tau, v_th, levels, 0.0, float(levels), False, False, 0,
                                                       recompute)
    assert v_seq.numel() == 0
    torch.autograd.backward([s, v_last], [gs.cuda(), gl.cuda()])
    torch.testing.assert_close(xd.grad.cpu(), ref["grad_x"], rtol=GRAD_RTOL, atol=GRAD_ATOL)
    torch.testing.assert_close(vd.grad.cpu(), ref["grad_v_init"], rtol=GRAD_RTOL, atol=GRAD_ATOL)
    s2, v_seq2, v_last2 = K.hip_multistep_ilif_inference(x.cuda(), v0.cuda(), tau, v_th, levels, True, 0)
    assert bits_equal(s2.cpu(), ref["spike_seq"]) and bits_equal(v_seq2.cpu(), ref["v_seq"])
    assert bits_equal(v_last2.cpu(), ref["v_seq"][-1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,N", [(8, 2048), (5, 77), (12, 8192)])
@pytest.mark.parametrize("tau,v_th,levels", [(1.6, 0.7, 4), (2.0, 1.0, 7), (4.0 / 3.0, 0.3, 3)])
def test_every_op_rounded_16bit_equals_torch_ops_on_half_tensors(K, dtype, T, N, tau, v_th, levels):
    """The torch backend on half tensors rounds after every op; a Python scalar stays fp32 in h / v_th and in
    count * v_th (two roundings: to fp32, then to the tensor dtype).  Counts, h and v must match bit for bit, and
    the gradients (whose window is tested on the rounded quotient) to 16-bit accuracy."""
    x = seeded_randn((T, N), 21, 0.6 * v_th * levels / 2, v_th * levels / 2).to(dtype)
    v0 = seeded_randn((N,), 22, 0.0, 0.3).to(dtype)
    gs = seeded_randn((T, N), 23).to(dtype)
    ref = no.forward_backward("ilif", x, v0, gs, None, None, tau, False, v_th, None, sg=no.multi_level_spike_count(levels))
    for recompute in ((False, True) if N % 8 == 0 else (False,)):
        xd, vd = x.cuda().requires_grad_(), v0.cuda().requires_grad_()
        s, v_seq, v_last, h = K.hip_multistep_ilif_forward(xd, vd, tau, v_th, levels, 0.0, float(levels), False, True, 0,
                                                           recompute)
        assert bits_equal(s.cpu(), ref["spike_seq"]) and bits_equal(v_seq.cpu(), ref["v_seq"])
        assert bits_equal(v_last.cpu(), ref["v_seq"][-1])
        if not recompute:
            assert bits_equal(h.cpu(), ref["h_seq"])
        s.backward(gs.cuda())
        # the oracle back-propagates in the 16-bit dtype, the kernel in fp32: compare against the size of the gradient
        err = (xd.grad.float().cpu() - ref["grad_x"].float()).abs().max()
        assert float(err) <= 3e-2 * float(ref["grad_x"].float().abs().max()) + 1e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fp32_state_16bit_storage(K, dtype):
    """fp32 state: inputs are 16-bit values, all arithmetic and the carried v are fp32, stored values are rounded
    (what the reference's Triton kernel does with compute_dtype fp32).  Counts are exact integers either way."""
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    T, N, tau, v_th, levels = 10, 4096, 1.6, 0.7, 4
    x = seeded_randn((T, N), 31, 0.8, 1.2).to(dtype)
    v0 = seeded_randn((N,), 32, 0.0, 0.3).to(dtype)
    gs = seeded_randn((T, N), 33).to(dtype)
    ref = no.forward_backward("ilif", x.float(), v0.float(), gs.float(), None, None, tau, False, v_th, None,
                              sg=no.multi_level_spike_count(levels))
    for recompute in (False, True):
        xd = x.cuda().requires_grad_()
        s, v_seq, v_last, _ = K.hip_multistep_ilif_forward(xd, v0.cuda(), tau, v_th, levels, 0.0, float(levels), False,
                                                           True, L.FLAG_FP32_STATE, recompute)
        assert bits_equal(s.cpu(), ref["spike_seq"].to(dtype))
        assert bits_equal(v_seq.cpu(), ref["v_seq"].to(dtype))
        assert bits_equal(v_last.cpu(), ref["v_seq"][-1].to(dtype))
        s.backward(gs.cuda())
        if recompute:  # h is exact in the replay; a stored h is rounded, which may move it across a window edge
            torch.testing.assert_close(xd.grad.float().cpu(), ref["grad_x"], rtol=1e-2, atol=1e-2)
        else:
            err = (xd.grad.float().cpu() - ref["grad_x"]).abs()
            assert float((err > 1e-2 + 1e-2 * ref["grad_x"].abs()).float().mean()) < 2e-3


def test_reference_known_answers_through_the_hip_backend():
    """Literal inputs and outputs of the reference's test/activation_based/test_ilif_node.py:336-344, 400-413,
    416-440, run with backend='hip'."""
    node = neuron.ILIFNode(v_threshold=1.0, tau=4.0 / 3.0, step_mode="m", backend="hip", store_v_seq=True)
    y = node(torch.tensor([[[3.2]], [[0.0]], [[4.8]], [[0.0]]]).cuda())
    assert torch.equal(y.flatten().cpu(), torch.tensor([3.0, 0.0, 4.0, 0.0]))
    assert node.v_seq.shape == y.shape
    node = neuron.ILIFNode(v_threshold=1.0, tau=4.0 / 3.0, step_mode="s", backend="hip")
    x = torch.tensor([[3.2, 0.4, 5.8]])
    y = node(x.cuda())
    assert torch.equal(y.cpu(), torch.tensor([[3.0, 0.0, 4.0]]))
    torch.testing.assert_close(node.v.cpu(), x - y.cpu())
    node = neuron.ILIFNode(v_threshold=1.0, step_mode="s", backend="hip")
    x = torch.tensor([[-0.5, 0.5, 4.5]]).cuda().requires_grad_()
    node(x).sum().backward()
    torch.testing.assert_close(x.grad.cpu(), torch.tensor([[0.0, 1.0, 0.0]]))
    node = neuron.ILIFNode(surrogate_function=surrogate.MultiLevelSpikeCount(4, grad_window=(-0.5, 4.5)), step_mode="s",
                           backend="hip")
    x = torch.tensor([[-0.25, 4.25, 4.75]]).cuda().requires_grad_()
    y = node(x)
    y.sum().backward()
    assert torch.equal(y.detach().cpu(), torch.tensor([[0.0, 4.0, 4.0]]))
    torch.testing.assert_close(x.grad.cpu(), torch.tensor([[1.0, 1.0, 0.0]]))


@pytest.mark.parametrize("detach_reset", [False, True])
@pytest.mark.parametrize("store_v_seq", [False, True])
def test_hip_node_matches_torch_node(detach_reset, store_v_seq):
    kw = dict(tau=1.6, v_threshold=0.7, surrogate_function=surrogate.MultiLevelSpikeCount(4),
              detach_reset=detach_reset, store_v_seq=store_v_seq)
    a = neuron.ILIFNode(step_mode="m", backend="torch", **kw)
    b = neuron.ILIFNode(step_mode="m", backend="hip", **kw).cuda()
    x = seeded_randn((6, 4, 12, 4), 20260501, 0.8, 1.2)
    xa, xb = x.clone().requires_grad_(), x.cuda().requires_grad_()
    sa, sb = a(xa), b(xb)
    (sa.sum() + 0.5 * a.v.sum()).backward()
    (sb.sum() + 0.5 * b.v.sum()).backward()
    assert float(sa.detach().max()) == 4.0
    assert bits_equal(sb.cpu(), sa.detach())
    assert bits_equal(b.v.detach().cpu(), a.v.detach())
    if store_v_seq:
        assert bits_equal(b.v_seq.detach().cpu(), a.v_seq.detach())
    torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=GRAD_RTOL, atol=GRAD_ATOL)
    # eval mode fires the same counts (no Heaviside swap for this neuron), and the state carries over
    a.eval()
    b.eval()
    with torch.no_grad():
        sa2, sb2 = a(x), b(x.cuda())
    assert bits_equal(sb2.cpu(), sa2) and float(sa2.max()) > 1.0
    functional.reset_net(a)
    functional.reset_net(b)


def test_half_precision_modes_of_the_node():
    old = configure.hip_half_precision_mode
    try:
        x = seeded_randn((8, 64, 32), 5, 0.8, 1.2).half()
        for mode in ("torch", "fp32_state"):
            configure.hip_half_precision_mode = mode
            node = neuron.ILIFNode(tau=1.6, v_threshold=0.7, step_mode="m", backend="hip")
            s = node(x.cuda())
            if mode == "torch":
                ref = neuron.ILIFNode(tau=1.6, v_threshold=0.7, step_mode="m", backend="torch")
                assert bits_equal(s.cpu(), ref(x))
            else:
                es, _, _ = no.multi_step("ilif", x.float().flatten(1), torch.zeros(64 * 32), 1.6, False, 0.7, None,
                                         no.multi_level_spike_count(4))
                assert bits_equal(s.cpu().flatten(1), es.half())
    finally:
        configure.hip_half_precision_mode = old
