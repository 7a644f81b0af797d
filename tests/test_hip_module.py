"""The drop-in boundary on the GPU: ``backend='hip'`` nodes against ``backend='torch'`` nodes and the
oracle, re-expressing the reference's own consistency tests (test_triton_neuron.py:671-766,
test_cupy_backend_comprehensive.py:316-424, test_compile_compat.py:380-493, 659-675)."""

import pytest
import torch

from oracle import neuron_oracle as no
from spikingjelly_amd import configure
from spikingjelly_amd.activation_based import functional, neuron, surrogate

from helpers import bits_equal, seeded_randn

pytestmark = pytest.mark.gpu

GRAD_RTOL, GRAD_ATOL = 1e-5, 1e-6


def _pair(cls, **kw):
    a = cls(step_mode="m", backend="torch", **kw)
    b = cls(step_mode="m", backend="hip", **kw).cuda()
    return a, b


def test_config1_lif_cpu_case():
    """BASELINE config 1: x [4,64,128] ~ N(0.5,1) seed 1001, grad_spike seed 1101, LIF tau=2, hard reset,
    ATan(2): spikes and h bit-exact, grad_x within 1e-5."""
    x = seeded_randn((4, 64, 128), 1001, 0.5, 1.0)
    gs = seeded_randn((4, 64, 128), 1101)
    ref = no.forward_backward("lif", x.flatten(1), torch.zeros(64 * 128), gs.flatten(1), None, None, 2.0, True, 1.0,
                              0.0, "atan", 2.0, False)
    node = neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(2.0), step_mode="m", backend="hip",
                          store_v_seq=True).cuda()
    xd = x.cuda().requires_grad_()
    s = node(xd)
    s.backward(gs.cuda())
    assert 0.05 < float(s.detach().mean()) < 0.15
    assert bits_equal(s.cpu().flatten(1), ref["spike_seq"])
    assert bits_equal(node.v_seq.detach().cpu().flatten(1), ref["v_seq"])
    assert bits_equal(node.v.detach().cpu().flatten(), ref["v_seq"][-1])
    torch.testing.assert_close(xd.grad.cpu().flatten(1), ref["grad_x"], rtol=GRAD_RTOL, atol=GRAD_ATOL)


@pytest.mark.parametrize("cls,kw", [
    (neuron.IFNode, {}),
    (neuron.LIFNode, {"tau": 2.0}),
    (neuron.LIFNode, {"tau": 5.0, "decay_input": False}),
    (neuron.ParametricLIFNode, {"init_tau": 2.0}),
    (neuron.ParametricLIFNode, {"init_tau": 2.0, "decay_input": False}),
])
@pytest.mark.parametrize("v_reset", [0.0, -0.2, None])
@pytest.mark.parametrize("detach_reset", [False, True])
@pytest.mark.parametrize("sg", [surrogate.ATan, surrogate.Sigmoid])
def test_hip_node_matches_torch_node(cls, kw, v_reset, detach_reset, sg):
    a, b = _pair(cls, v_threshold=0.5, v_reset=v_reset, detach_reset=detach_reset, surrogate_function=sg(), **kw)
    x = seeded_randn((6, 4, 12, 4), 20260428, 0.3, 1.0)
    xa = x.clone().requires_grad_()
    xb = x.cuda().requires_grad_()
    sa, sb = a(xa), b(xb)
    (sa.sum() + 0.5 * a.v.sum()).backward()
    (sb.sum() + 0.5 * b.v.sum()).backward()
    assert bits_equal(sb.cpu(), sa.detach())
    assert bits_equal(b.v.detach().cpu(), a.v.detach())
    torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=GRAD_RTOL, atol=GRAD_ATOL)
    if cls is neuron.ParametricLIFNode:
        torch.testing.assert_close(b.w.grad.cpu(), a.w.grad, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("decay_input", [True, False])
@pytest.mark.parametrize("v_reset", [0.0, -0.2, None])
def test_reciprocal_tau_switch_matches_the_torch_backend_on_the_same_device(decay_input, v_reset, monkeypatch):
    """tau = 3 is not a power of two.  torch divides a device tensor by a Python scalar as a multiplication by 1/tau,
    which is also what the reference's CuPy / Triton kernels are handed (multi_step/lif.py:338); with
    ``configure.hip_lif_reciprocal_tau = True`` the hip backend fires the same spikes as ``backend='torch'`` run on the
    GPU, while the default (IEEE division) fires the spikes of ``backend='torch'`` run on the CPU."""
    x = seeded_randn((8, 64, 257), 31, 0.4, 1.0)
    kw = dict(tau=3.0, decay_input=decay_input, v_reset=v_reset, surrogate_function=surrogate.ATan(), step_mode="m")
    on_gpu = neuron.LIFNode(backend="torch", store_v_seq=True, **kw).cuda()
    s_gpu = on_gpu(x.cuda())
    on_cpu = neuron.LIFNode(backend="torch", store_v_seq=True, **kw)
    s_cpu = on_cpu(x)
    for flag, s_ref, node_ref in ((True, s_gpu, on_gpu), (False, s_cpu, on_cpu)):
        monkeypatch.setattr(configure, "hip_lif_reciprocal_tau", flag)
        node = neuron.LIFNode(backend="hip", store_v_seq=True, **kw).cuda()
        s = node(x.cuda())
        assert bits_equal(s.cpu(), s_ref.cpu()), flag
        assert bits_equal(node.v_seq.cpu(), node_ref.v_seq.cpu()), flag
    assert not bits_equal(on_gpu.v_seq.cpu(), on_cpu.v_seq)  # the two torch runs really differ on this input


@pytest.mark.parametrize("cls", [neuron.IFNode, neuron.LIFNode, neuron.ParametricLIFNode])
@pytest.mark.parametrize("T,N", [(1, 48), (7, 111), (65, 64)])
def test_store_v_seq_toggle_is_equivalent(cls, T, N):
    x = seeded_randn((T, 2, N), 5, 0.4, 1.0).cuda()
    gs, gv = seeded_randn((T, 2, N), 6).cuda(), seeded_randn((2, N), 7).cuda()
    outs = []
    for store in (False, True):
        node = cls(step_mode="m", backend="hip", store_v_seq=store, surrogate_function=surrogate.ATan()).cuda()
        xi = x.clone().requires_grad_()
        s = node(xi)
        ((s * gs).sum() + (node.v * gv).sum()).backward()
        if store:
            assert node.v_seq.shape == x.shape and bits_equal(node.v_seq[-1].detach(), node.v.detach())
        else:
            assert node.v_seq is None
        outs.append((s.detach(), node.v.detach(), xi.grad))
    for u, w in zip(*outs):
        assert bits_equal(u, w)


@pytest.mark.parametrize("cls", [neuron.IFNode, neuron.LIFNode, neuron.ParametricLIFNode])
@pytest.mark.parametrize("N,store_v_seq", [(64, False), (64, True), (37, False), (37, True)])  # replay and saved-h kernels
def test_loss_on_the_membrane_potential_alone(cls, N, store_v_seq):
    """No gradient reaches the spikes: the kernels are handed no spike gradient at all (nothing is allocated, filled
    or read in its place) and must give the gradients of the torch backend."""
    x = seeded_randn((6, 3, N), 12, 0.4, 1.0)
    gv = seeded_randn((6, 3, N) if store_v_seq else (3, N), 13)
    a, b = _pair(cls, surrogate_function=surrogate.ATan(), store_v_seq=store_v_seq)
    xa, xb = x.clone().requires_grad_(), x.cuda().requires_grad_()
    a(xa)
    b(xb)
    ((a.v_seq if store_v_seq else a.v) * gv).sum().backward()
    ((b.v_seq if store_v_seq else b.v) * gv.cuda()).sum().backward()
    torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=GRAD_RTOL, atol=GRAD_ATOL)
    if cls is neuron.ParametricLIFNode:
        torch.testing.assert_close(b.w.grad.cpu(), a.w.grad, rtol=1e-4, atol=1e-5)


def test_non_contiguous_upstream_gradient():
    x = seeded_randn((8, 16, 32), 8, 0.4, 1.0)
    a, b = _pair(neuron.LIFNode, surrogate_function=surrogate.ATan())
    xa, xb = x.clone().requires_grad_(), x.cuda().requires_grad_()
    g = seeded_randn((32, 16, 8), 9).permute(2, 1, 0)
    assert not g.is_contiguous()
    a(xa).backward(g)
    b(xb).backward(g.cuda())
    torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=GRAD_RTOL, atol=GRAD_ATOL)


def test_v_init_gradient_and_user_assigned_state():
    x = seeded_randn((5, 3, 40), 10, 0.4, 1.0)
    v0 = seeded_randn((3, 40), 11, 0.0, 0.3)
    a, b = _pair(neuron.LIFNode, tau=2.5, surrogate_function=surrogate.Sigmoid())
    va, vb = v0.clone().requires_grad_(), v0.cuda().requires_grad_()
    a.v, b.v = va, vb
    sa, sb = a(x), b(x.cuda())
    (sa.sum() + a.v.sum()).backward()
    (sb.sum() + b.v.sum()).backward()
    assert bits_equal(sb.cpu(), sa.detach())
    torch.testing.assert_close(vb.grad.cpu(), va.grad, rtol=GRAD_RTOL, atol=GRAD_ATOL)


def test_state_carries_over_and_batch_size_change_reinitialises():
    a, b = _pair(neuron.LIFNode, surrogate_function=surrogate.ATan())
    x1, x2 = seeded_randn((4, 8, 16), 12, 0.4, 1.0), seeded_randn((4, 8, 16), 13, 0.4, 1.0)
    for x in (x1, x2):  # second call continues from the first call's v
        assert bits_equal(b(x.cuda()).cpu(), a(x))
    x3 = seeded_randn((4, 3, 16), 14, 0.4, 1.0)  # batch size changed without reset
    assert bits_equal(b(x3.cuda()).cpu(), a(x3))
    functional.reset_net(a)
    functional.reset_net(b)
    assert b.v == 0.0 and isinstance(b.v, float)
    assert bits_equal(b(x1.cuda()).cpu(), a(x1))


@pytest.mark.parametrize("ctx", ["eval", "no_grad", "inference_mode"])
def test_inference_modes(ctx):
    a, b = _pair(neuron.IFNode, v_reset=None, surrogate_function=surrogate.ATan())
    x = seeded_randn((6, 4, 32), 15, 0.3, 0.5)
    if ctx == "eval":
        a.eval()
        b.eval()
        sa, sb = a(x), b(x.cuda())
    else:
        cm = torch.no_grad if ctx == "no_grad" else torch.inference_mode
        with cm():
            sa, sb = a(x), b(x.cuda())
    assert bits_equal(sb.cpu(), sa) and bits_equal(b.v.cpu(), a.v)


def test_training_after_a_first_forward_under_inference_mode():
    """The shared one-element initial state (one per device, dtype and value; -0.37 is used by no other test) is first
    made under ``torch.inference_mode()``: a later training forward saves its expanded view for the backward, which an
    inference tensor would refuse."""
    kw = dict(v_reset=-0.37, surrogate_function=surrogate.ATan())
    x = seeded_randn((6, 4, 32), 16, 0.3, 0.5)
    first = neuron.LIFNode(step_mode="m", backend="hip", **kw).cuda()
    with torch.inference_mode():
        first(x.cuda())
    a, b = _pair(neuron.LIFNode, **kw)
    xa, xb = x.clone().requires_grad_(), x.cuda().requires_grad_()
    sa, sb = a(xa), b(xb)
    g = seeded_randn(sa.shape, 17)
    sa.backward(g)
    sb.backward(g.cuda())
    assert bits_equal(sb.detach().cpu(), sa.detach())
    torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=GRAD_RTOL, atol=GRAD_ATOL)


def test_unsupported_surrogate_and_primitive_mode_raise():
    node = neuron.LIFNode(step_mode="m", backend="hip", surrogate_function=surrogate.PiecewiseLeakyReLU()).cuda()
    x = torch.randn(4, 2, 8, device="cuda", requires_grad=True)
    with pytest.raises(NotImplementedError, match="PiecewiseLeakyReLU"):
        node(x)
    node = neuron.LIFNode(step_mode="m", backend="hip", surrogate_function=surrogate.ATan(spiking=False)).cuda().eval()
    with pytest.raises(NotImplementedError, match="spiking"):
        node(x)
    with pytest.raises(NotImplementedError):
        neuron.LIFNode(step_mode="m", backend="hip")(torch.randn(4, 2, 8, device="cuda", dtype=torch.float64))


def test_cpu_tensor_is_rejected_not_silently_computed():
    node = neuron.LIFNode(step_mode="m", backend="hip")
    with pytest.raises(RuntimeError, match="ROCm device"):
        node(torch.randn(4, 2, 8))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("cls", [neuron.IFNode, neuron.LIFNode, neuron.ParametricLIFNode])
def test_half_nodes_match_torch_backend_bitwise(dtype, cls):
    a, b = _pair(cls, v_reset=None, surrogate_function=surrogate.Sigmoid())
    x = seeded_randn((8, 4, 64), 16, 0.3, 1.0).to(dtype)
    with torch.no_grad():
        sa, sb = a(x), b(x.cuda())
    assert sb.dtype == dtype and bits_equal(sb.cpu(), sa) and bits_equal(b.v.cpu(), a.v)


def test_fp32_state_mode_for_bf16_plif():
    """Config-3 semantics: bf16 storage, fp32 state; oracle = the reference's mixed-precision recipe."""
    x = seeded_randn((8, 4, 256), 1003, 0.2, 1.0).bfloat16()
    es, ev, _ = no.multi_step_mixed_precision("plif", x.float().flatten(1), torch.zeros(4 * 256), torch.bfloat16, 0.5,
                                              True, 1.0, None)
    node = neuron.ParametricLIFNode(init_tau=2.0, v_reset=None, step_mode="m", backend="hip", store_v_seq=True).cuda()
    old = configure.hip_half_precision_mode
    configure.hip_half_precision_mode = "fp32_state"
    try:
        with torch.no_grad():
            s = node(x.cuda())
    finally:
        configure.hip_half_precision_mode = old
    assert torch.equal(s.cpu().float().flatten(1), es)
    assert torch.equal(node.v_seq.cpu().float().flatten(1), ev)


def test_set_backend_switches_supported_modules_only():
    net = torch.nn.Sequential(neuron.LIFNode(step_mode="m"), torch.nn.Linear(4, 4), neuron.IFNode(step_mode="s"))
    functional.set_backend(net, "hip")
    assert net[0].backend == "hip" and net[2].backend == "hip" and not hasattr(net[1], "backend")


@pytest.mark.parametrize("cls,kw", [
    (neuron.IFNode, {}),
    (neuron.LIFNode, {"tau": 3.0}),
    (neuron.LIFNode, {"tau": 2.0, "decay_input": False}),
    (neuron.ParametricLIFNode, {"init_tau": 2.0}),
])
@pytest.mark.parametrize("v_reset", [0.0, None])
@pytest.mark.parametrize("detach_reset", [False, True])
def test_single_step_hip_loop_matches_multi_step_torch(cls, kw, v_reset, detach_reset):
    """step_mode='s' with backend='hip' (the reference's single-step kernel backends,
    functional/neuron.py:1709-1886): a Python loop over T single steps, state and its gradient carried
    through self.v between kernel calls, equals the torch backend's multi-step run."""
    T = 5
    a = cls(step_mode="m", backend="torch", v_threshold=0.5, v_reset=v_reset, detach_reset=detach_reset,
            surrogate_function=surrogate.ATan(), **kw)
    b = cls(step_mode="s", backend="hip", v_threshold=0.5, v_reset=v_reset, detach_reset=detach_reset,
            surrogate_function=surrogate.ATan(), **kw).cuda()
    x = seeded_randn((T, 3, 40), 77, 0.3, 1.0)
    g = seeded_randn((T, 3, 40), 78)
    xa, xb = x.clone().requires_grad_(), x.cuda().requires_grad_()
    sa = a(xa)
    sb = torch.stack([b(xb[t]) for t in range(T)])
    assert bits_equal(sb.cpu(), sa.detach())
    assert bits_equal(b.v.detach().cpu(), a.v.detach())
    ((sa * g).sum() + 0.5 * a.v.sum()).backward()
    ((sb * g.cuda()).sum() + 0.5 * b.v.sum()).backward()
    torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=GRAD_RTOL, atol=GRAD_ATOL)
    if cls is neuron.ParametricLIFNode:
        torch.testing.assert_close(b.w.grad.cpu(), a.w.grad, rtol=1e-4, atol=1e-5)


def test_single_step_functionals_return_spike_and_state():
    x = seeded_randn((4, 33), 79, 0.6, 1.0).cuda()
    v = torch.zeros_like(x)
    es, ev, _ = no.multi_step("lif", x.cpu().unsqueeze(0), v.cpu(), 2.0, True, 1.0, 0.0)
    s, v_next = functional.lif_step_hip(x, v, 2.0, True, 1.0, 0.0, surrogate.ATan())
    assert s.shape == x.shape and v_next.shape == x.shape
    assert bits_equal(s.cpu(), es[0]) and bits_equal(v_next.cpu(), ev[0])
    s, v_next = functional.if_step_hip(x, v, 1.0, None, surrogate.Sigmoid())
    es, ev, _ = no.multi_step("if", x.cpu().unsqueeze(0), v.cpu(), None, True, 1.0, None)
    assert bits_equal(s.cpu(), es[0]) and bits_equal(v_next.cpu(), ev[0])


@pytest.mark.parametrize("cls", [neuron.IFNode, neuron.LIFNode, neuron.ParametricLIFNode])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_replay_and_h_seq_backward_paths_agree(cls, dtype):
    """configure.hip_backward_recompute only changes where h comes from in the backward (replayed from x
    vs read from a saved h_seq); in fp32 both see the same h bit for bit, so gradients must be identical."""
    x = seeded_randn((16, 4, 256), 31, 0.4, 1.0).to(dtype).cuda()
    gs = seeded_randn((16, 4, 256), 32).to(dtype).cuda()
    grads = []
    old = configure.hip_backward_recompute
    try:
        for flag in (True, False):
            configure.hip_backward_recompute = flag
            node = cls(step_mode="m", backend="hip", surrogate_function=surrogate.ATan(), store_v_seq=True).cuda()
            xi = x.clone().requires_grad_()
            s = node(xi)
            (s * gs).sum().backward()
            grads.append((s.detach(), node.v_seq.detach(), xi.grad))
    finally:
        configure.hip_backward_recompute = old
    assert bits_equal(grads[0][0], grads[1][0]) and bits_equal(grads[0][1], grads[1][1])
    if dtype == torch.float32:
        assert bits_equal(grads[0][2], grads[1][2])
    else:
        torch.testing.assert_close(grads[0][2].float(), grads[1][2].float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("cls", [neuron.IFNode, neuron.LIFNode, neuron.ParametricLIFNode, neuron.QIFNode])
@pytest.mark.parametrize("T", [40, 64, 100, 128])
@pytest.mark.parametrize("store_v_seq", [False, True])
def test_long_sequences_replayed_in_pieces_equal_the_saved_h_route(cls, T, store_v_seq, monkeypatch):
    """Beyond the length the replay kernel takes in one piece the forward leaves the state every
    ``configure.hip_replay_chunk`` steps and the backward replays piece by piece from those checkpoints; with the
    chunking switched off the same sequence saves and reads h_seq.  fp32: spikes and states identical bit for bit; the
    gradient crosses a piece boundary as an fp32 tensor, so the two routes perform the same operations and differ at
    most where the compiler fused a multiply-add in one kernel variant and not in the other (a short last piece runs
    the short-sequence variant): 1e-6 relative.  The PLIF sum is added in another order."""
    from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K

    x = seeded_randn((T, 2, 512), 33, 0.4, 1.0).cuda()
    gs = seeded_randn((T, 2, 512), 34).cuda()
    gv = seeded_randn((T, 2, 512) if store_v_seq else (2, 512), 35, 0.0, 0.2).cuda()
    v0 = seeded_randn((2, 512), 36, 0.0, 0.3).cuda()
    pieces = []
    real = K._run_backward
    monkeypatch.setattr(K, "_run_backward", lambda *a, **k: (pieces.append(a[17]), real(*a, **k))[1])
    results = []
    for chunk in (16, 0):
        monkeypatch.setattr(configure, "hip_replay_chunk", chunk)
        node = cls(step_mode="m", backend="hip", surrogate_function=surrogate.ATan(), store_v_seq=store_v_seq).cuda()
        vi = v0.clone().requires_grad_()
        node.v = vi
        xi = x.clone().requires_grad_()
        s = node(xi)
        ((s * gs).sum() + ((node.v_seq if store_v_seq else node.v) * gv).sum()).backward()
        results.append((s.detach(), node.v.detach(), xi.grad, vi.grad, node.w.grad if hasattr(node, "w") else None))
    assert pieces == [16, 0]  # the first run was chunked, the second was not
    for a, b in zip(results[0][:2], results[1][:2]):
        assert bits_equal(a, b)
    for a, b in zip(results[0][2:4], results[1][2:4]):
        torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-7)
    if results[0][4] is not None:
        torch.testing.assert_close(results[0][4], results[1][4], rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("cls", [neuron.IFNode, neuron.LIFNode, neuron.ParametricLIFNode])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=lambda v: str(v).replace("torch.", ""))
@pytest.mark.parametrize("T", [64, 100])
def test_long_16_bit_sequences_with_fp32_state_are_replayed_in_pieces(cls, dtype, T, monkeypatch):
    """16-bit storage with the state kept in fp32: the checkpoints are fp32, so the forward in pieces equals the plain
    forward bit for bit, and the backward (which replays the unrounded h) is the same at two piece lengths; the PLIF
    sum is added in another order."""
    from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K

    monkeypatch.setattr(configure, "hip_half_precision_mode", "fp32_state")
    x = seeded_randn((T, 2, 512), 43, 0.4, 1.0).to(dtype).cuda()
    gs = seeded_randn((T, 2, 512), 44).to(dtype).cuda()
    gv = seeded_randn((2, 512), 45, 0.0, 0.2).to(dtype).cuda()
    v0 = seeded_randn((2, 512), 46, 0.0, 0.3).to(dtype).cuda()
    pieces = []
    real = K._run_backward
    monkeypatch.setattr(K, "_run_backward", lambda *a, **k: (pieces.append(a[17]), real(*a, **k))[1])
    results = []
    for chunk in (16, 32, 0):
        monkeypatch.setattr(configure, "hip_replay_chunk", chunk)
        node = cls(step_mode="m", backend="hip", surrogate_function=surrogate.ATan()).cuda()
        vi = v0.clone().requires_grad_()
        node.v = vi
        xi = x.clone().requires_grad_()
        s = node(xi)
        ((s * gs).sum() + (node.v * gv).sum()).backward()
        results.append((s.detach(), node.v.detach(), xi.grad, vi.grad, node.w.grad if hasattr(node, "w") else None))
    assert pieces == [16, 32, 0]
    for other in results[1:]:
        assert bits_equal(results[0][0], other[0]) and bits_equal(results[0][1], other[1])
    assert bits_equal(results[0][2], results[1][2]) and bits_equal(results[0][3], results[1][3])
    assert not torch.isnan(results[0][2].float()).any() and float(results[0][2].float().abs().sum()) > 0
    if results[0][4] is not None:
        torch.testing.assert_close(results[0][4], results[1][4], rtol=1e-4, atol=1e-5)


def test_long_sequence_in_pieces_matches_the_torch_backend():
    x = seeded_randn((70, 3, 64), 37, 0.4, 1.0)
    gs = seeded_randn((70, 3, 64), 38)
    a, b = _pair(neuron.LIFNode, tau=2.5, v_reset=-0.1, surrogate_function=surrogate.Sigmoid())
    xa, xb = x.clone().requires_grad_(), x.cuda().requires_grad_()
    sa, sb = a(xa), b(xb)
    (sa * gs).sum().backward()
    (sb * gs.cuda()).sum().backward()
    assert bits_equal(sb.cpu(), sa.detach()) and bits_equal(b.v.detach().cpu(), a.v.detach())
    torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=GRAD_RTOL, atol=GRAD_ATOL)


def test_replay_path_with_misaligned_and_non_contiguous_input():
    """A sliced (16-byte misaligned) x_seq and a permuted upstream gradient still take the replay path."""
    base = seeded_randn((8, 4, 65), 33, 0.4, 1.0)
    x = base[:, :, 1:]  # [8,4,64] view, rows start 4 bytes off
    a, b = _pair(neuron.LIFNode, surrogate_function=surrogate.ATan())
    xa, xb = x.clone().requires_grad_(), base.cuda()[:, :, 1:].requires_grad_()
    g = seeded_randn((64, 4, 8), 34).permute(2, 1, 0)
    a(xa).backward(g)
    b(xb).backward(g.cuda())
    torch.testing.assert_close(xb.grad.cpu(), xa.grad, rtol=GRAD_RTOL, atol=GRAD_ATOL)



@pytest.mark.gpu
def test_matrix_core_probe_runs_and_refuses_bad_arguments():
    """sjhip_mfma_probe (no counterpart in the reference: the ceiling bench.py holds the convolution GEMMs against) performs
    the flops it reports, writes one float per block and rejects what it cannot launch."""
    from spikingjelly_amd.activation_based.hip_kernel import library as L
    lib = L.load()
    blocks = lib.sjhip_mfma_probe_blocks(1)
    assert blocks >= 1 and lib.sjhip_mfma_probe_blocks(2) == 2 * blocks and lib.sjhip_mfma_probe_blocks(0) == 0
    sink = torch.full((2 * blocks,), float("nan"), device="cuda:0")
    L.profile_reset()
    L.profile_enable(True)
    flop_zero = L.mfma_probe(False, 1, 500, sink)
    flop_random = L.mfma_probe(True, 2, 500, sink)
    torch.cuda.synchronize()
    L.profile_enable(False)
    n, ms = L.profile_read(L.KC_MFMA_PROBE)
    assert n == 2 and ms > 0.0
    assert flop_zero == blocks * 4 * 500 * 16 * 32768 and flop_random == 2 * flop_zero
    assert torch.isfinite(sink).all()  # every block of the larger launch wrote its float
    tflops = (flop_zero + flop_random) / (ms * 1e-3) / 1e12
    assert 100.0 < tflops < 2600.0, tflops  # between a tenth of and the published fp16 peak of an MI355X
    st = L.current_stream_ptr(torch.device("cuda:0"))
    for bad in [(2, 1, 10, sink.data_ptr(), sink.numel()), (0, 0, 10, sink.data_ptr(), sink.numel()), (0, 9, 10, sink.data_ptr(), sink.numel()),
                (0, 1, 0, sink.data_ptr(), sink.numel()), (0, 1, 10, None, sink.numel()), (0, 1, 10, sink.data_ptr(), blocks - 1)]:
        assert lib.sjhip_mfma_probe(*bad, st) != 0
