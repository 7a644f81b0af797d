"""``torch.compile(..., fullgraph=True)`` over modules with ``backend='hip'``: the kernels are opaque operators with
fake (meta) implementations, and everything the host side does around them must be traceable without a graph break,
as the reference requires of its kernel backends (test/activation_based/test_compile_compat.py:125-170, 496-525).
The ``aot_eager`` backend traces forward and backward through AOT autograd and then runs the graph with the eager
kernels, so results must equal the uncompiled module exactly."""

import pytest
import torch

from spikingjelly_amd.activation_based import layer, neuron, surrogate

from helpers import seeded_randn

pytestmark = pytest.mark.gpu

NODES = {
    "if": lambda **kw: neuron.IFNode(surrogate_function=surrogate.ATan(), **kw),
    "lif": lambda **kw: neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(), **kw),
    "lif_soft_div": lambda **kw: neuron.LIFNode(tau=3.0, v_reset=None, decay_input=False,
                                                surrogate_function=surrogate.Sigmoid(), **kw),
    "plif": lambda **kw: neuron.ParametricLIFNode(surrogate_function=surrogate.ATan(), **kw),
    "qif": lambda **kw: neuron.QIFNode(tau=2.0, surrogate_function=surrogate.ATan(), **kw),
    "eif": lambda **kw: neuron.EIFNode(tau=2.0, surrogate_function=surrogate.ATan(), **kw),
    "ilif": lambda **kw: neuron.ILIFNode(**kw),
    "izhikevich": lambda **kw: neuron.IzhikevichNode(a=0.3, b=0.2, tau_w=3.0, surrogate_function=surrogate.ATan(), **kw),
}


@pytest.fixture(autouse=True)
def fresh_tracer():
    # every node class shares the code object of MemoryModule.forward, and the recompile limit is per code object
    torch._dynamo.reset()
    yield
    torch._dynamo.reset()


def _compiled(module):
    return torch.compile(module, fullgraph=True, backend="aot_eager")


@pytest.mark.parametrize("kind", sorted(NODES))
@pytest.mark.parametrize("store_v_seq", [False, True])
def test_multi_step_node_compiles_without_graph_breaks(kind, store_v_seq):
    scale = {"qif": 0.4, "eif": 0.5, "ilif": 2.0, "izhikevich": 0.5}.get(kind, 0.8)
    x = (seeded_randn((6, 4, 32), 11, 0.3, scale)).cuda()
    eager = NODES[kind](step_mode="m", backend="hip", store_v_seq=store_v_seq).cuda()
    traced = NODES[kind](step_mode="m", backend="hip", store_v_seq=store_v_seq).cuda()
    fn = _compiled(traced)
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    ya, yb = eager(xa), fn(xb)
    assert torch.equal(ya, yb) and float(ya.detach().abs().sum()) > 0
    assert torch.equal(eager.v, traced.v)
    if store_v_seq:
        assert torch.equal(eager.v_seq, traced.v_seq)
    (ya.sum() + 0.5 * eager.v.sum()).backward()
    (yb.sum() + 0.5 * traced.v.sum()).backward()
    assert torch.equal(xa.grad, xb.grad)
    if kind == "plif":
        torch.testing.assert_close(traced.w.grad, eager.w.grad)
    # the state is an ordinary tensor now: the second call re-traces once and continues from it
    assert torch.equal(eager(x), fn(x)) and torch.equal(eager.v, traced.v)


def test_inference_single_step_and_changing_shapes():
    """Eval mode, step_mode='s', and a sequence of different shapes (the tracer then treats sizes as symbols: the
    host-side policy around the operators must stay traceable)."""
    node = neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(), step_mode="m", backend="hip").cuda().eval()
    fn = _compiled(node)
    ref = neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(), step_mode="m", backend="hip").cuda().eval()
    for shape in ((6, 4, 32), (3, 8, 16), (5, 2, 20), (40, 2, 8), (41, 2, 8)):
        x = seeded_randn(shape, sum(shape), 0.3, 0.8).cuda()
        node.reset()
        ref.reset()
        with torch.no_grad():
            assert torch.equal(fn(x), ref(x))
    train = neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(), step_mode="m", backend="hip").cuda()
    fn = _compiled(train)
    for shape in ((6, 4, 32), (3, 8, 16), (5, 2, 20), (39, 2, 8), (40, 2, 8)):  # 39 / 40: either side of the replay limit
        x = seeded_randn(shape, sum(shape), 0.3, 0.8).cuda().requires_grad_()
        train.reset()
        fn(x).sum().backward()
        assert bool(torch.isfinite(x.grad).all()) and float(x.grad.abs().sum()) > 0
    single = neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(), step_mode="s", backend="hip").cuda()
    fn = _compiled(single)
    ref = neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(), step_mode="s", backend="hip").cuda()
    x = seeded_randn((4, 64), 3, 0.6, 0.8).cuda()
    for _ in range(3):
        assert torch.equal(fn(x), ref(x))


def test_spiking_self_attention_block_compiles():
    def make(backend):
        torch.manual_seed(1)
        block = layer.SpikingSelfAttention(128, 4, backend=backend).cuda()
        with torch.no_grad():  # freshly initialised, the block hardly fires: raise the batch-norm gains
            block.qkv_conv_bn[1].weight.fill_(2.0)
            block.proj_conv_bn[1].weight.fill_(3.0)
        return block

    x = seeded_randn((4, 8, 128, 96), 5).cuda()  # large enough for the attention LIF to receive coincident spikes
    eager, traced, torch_traced = make("hip"), make("hip"), make("torch")
    fn, fn_torch = _compiled(traced), _compiled(torch_traced)
    xa, xb, xc = (x.clone().requires_grad_() for _ in range(3))
    ya, yb, yc = eager(xa), fn(xb), fn_torch(xc)
    assert float(ya.detach().mean()) > 0.05
    assert torch.equal(ya, yb) and torch.equal(yb, yc)
    ya.sum().backward()
    yb.sum().backward()
    yc.sum().backward()
    torch.testing.assert_close(xb.grad, xa.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(xb.grad, xc.grad, rtol=1e-3, atol=1e-4)


def _triton_available() -> bool:
    try:
        import triton  # noqa: F401
    except Exception:
        return False
    return True


@pytest.mark.skipif(not _triton_available(), reason="the inductor backend generates triton kernels and triton is not importable")
@pytest.mark.parametrize("shape", [(4, 8, 32), (6, 3, 48)])
def test_inductor_compiles_linear_then_hip_node(shape):
    """Linear -> multi-step hip LIF -> loss under the code-generating backend, forward and backward, as the reference
    asks of its kernel backends (test/activation_based/test_compile_compat.py:144-170): the generated code around the
    opaque operators must hand them contiguous tensors and accept their outputs.  The linear layer runs through
    generated or library GEMM code, so its output may differ from eager in the last bit and a neuron at the threshold
    may flip: spikes are compared as a rate of disagreement, gradients with a tolerance."""
    T, B, D = shape

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = torch.nn.Linear(D, 2 * D)
            self.node = neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(), step_mode="m", backend="hip")

        def forward(self, x):
            return self.node(self.fc(x))

    torch.manual_seed(3)
    eager = Net().cuda()
    traced = Net().cuda()
    traced.load_state_dict(eager.state_dict())
    fn = torch.compile(traced, fullgraph=True, backend="inductor")
    x = seeded_randn((T, B, D), 17, 0.2, 1.5).cuda()
    target = seeded_randn((T, B, 2 * D), 18).cuda()
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    ya, yb = eager(xa), fn(xb)
    assert ya.shape == yb.shape == (T, B, 2 * D)
    assert 0.02 < float(ya.detach().mean()) < 0.9
    assert float((ya != yb).float().mean()) < 1e-3
    ((ya - target) ** 2).mean().backward()
    ((yb - target) ** 2).mean().backward()
    scale = float(xa.grad.abs().max())
    assert scale > 0
    torch.testing.assert_close(xb.grad, xa.grad, rtol=1e-3, atol=1e-3 * scale)
    torch.testing.assert_close(traced.fc.weight.grad, eager.fc.weight.grad, rtol=1e-3,
                               atol=1e-3 * float(eager.fc.weight.grad.abs().max()))


def _attention_block(dim, heads, seed, parametric=False):
    torch.manual_seed(seed)
    block = layer.SpikingSelfAttention(dim, heads, backend="hip")
    if parametric:  # the neurons at the end of the two chains learn their time constant
        block.qkv_lif = neuron.ParametricLIFNode(init_tau=2.5, step_mode="m", backend="hip")
        block.proj_lif = neuron.ParametricLIFNode(init_tau=3.0, step_mode="m", backend="hip")
    block = block.cuda().train()
    with torch.no_grad():
        block.qkv_conv_bn[1].weight.fill_(2.0)
        block.proj_conv_bn[1].weight.fill_(3.0)
    return block


def _launch_counts(L):
    return {name: L.profile_read(getattr(L, name))[0] for name in
            ("KC_PW_GEMM", "KC_PW_GRAD_WEIGHT", "KC_BN_LIF_FORWARD", "KC_BN_LIF_BACKWARD", "KC_BN_GRAD_INPUT", "KC_SSA_FORWARD",
             "KC_SSA_BACKWARD", "KC_FORWARD", "KC_BACKWARD")}


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
@pytest.mark.parametrize("dim,heads,T,B,tokens,parametric", [(64, 2, 4, 2, 36, False), (384, 12, 4, 2, 196, False),
                                                             (64, 2, 4, 2, 36, True)])
def test_compiled_attention_block_keeps_the_fused_chain(backend, dim, heads, T, B, tokens, parametric):
    """``torch.compile(SpikingSelfAttention(..., backend='hip'), fullgraph=True)`` launches the kernels of the fused
    convolution / batch norm / LIF chain that the eager module launches (counted by the library's own launch counters:
    the convolution GEMMs, the batch-norm + LIF kernels, the contraction), in forward and backward, with results equal
    to eager bit for bit: the chain is a set of opaque operators to the tracer, as the reference's kernel backends are
    (test/activation_based/test_compile_compat.py:125-170)."""
    from spikingjelly_amd.activation_based import functional
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    if backend == "inductor" and not _triton_available():
        pytest.skip("the inductor backend generates triton kernels and triton is not importable")
    eager, traced = _attention_block(dim, heads, 7, parametric), _attention_block(dim, heads, 7, parametric)
    fn = torch.compile(traced, fullgraph=True, backend=backend)
    x = seeded_randn((T, B, dim, tokens), 19).cuda()
    g = seeded_randn((T, B, dim, tokens), 20).cuda()
    results = []
    for module, call in ((eager, eager), (traced, fn)):
        xi = x.clone().requires_grad_()
        call(xi).backward(g)  # (first call: compilation; its launches are not counted; both modules take the same step)
        functional.reset_net(module)
        module.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_()
        torch.cuda.synchronize()
        L.profile_reset()
        L.profile_enable(True)
        out = call(xi)
        out.backward(g)
        torch.cuda.synchronize()
        L.profile_enable(False)
        results.append((out.detach(), xi.grad, [p.grad for p in module.parameters()], _launch_counts(L),
                        [b.clone() for b in module.buffers()]))
        functional.reset_net(module)
    (out_e, gx_e, gp_e, counts_e, buf_e), (out_c, gx_c, gp_c, counts_c, buf_c) = results
    assert counts_e["KC_PW_GEMM"] == 4 and counts_e["KC_PW_GRAD_WEIGHT"] == 2 and counts_e["KC_BN_LIF_FORWARD"] == 2
    assert counts_c == counts_e, (counts_c, counts_e)
    assert float(out_e.mean()) > 0.02
    assert torch.equal(out_c, out_e) and torch.equal(gx_c, gx_e)
    for a, b in zip(gp_c, gp_e):
        if a.dim() == 0:  # a parametric LIF's w: dL/dk times the sigmoid's derivative, which the code generator may fuse
            torch.testing.assert_close(a, b, rtol=1e-5, atol=0.0)
        else:
            assert torch.equal(a, b)
    for a, b in zip(buf_c, buf_e):   # running statistics and the batch counter
        assert torch.equal(a, b)
    if parametric:
        assert abs(float(eager.qkv_lif.w.grad)) > 0 and abs(float(eager.proj_lif.w.grad)) > 0
