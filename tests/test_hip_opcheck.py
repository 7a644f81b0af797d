"""``torch.library.opcheck`` on the operators of the hip backend: schema, fake (meta) kernels, autograd
registration and AOT dispatch must be consistent with what the real kernels return, so the ops can be traced
the way the reference's ``sj::`` operators are (test_compile_compat.py:125-170, 496-525)."""

import pytest
import torch

from helpers import seeded_randn

pytestmark = pytest.mark.gpu

TESTS = ("test_schema", "test_faketensor", "test_autograd_registration", "test_aot_dispatch_dynamic")


@pytest.fixture(scope="module")
def K():
    from spikingjelly_amd.activation_based.hip_kernel import library, neuron_kernel

    library.load()
    return neuron_kernel


@pytest.mark.parametrize("recompute", [False, True])
@pytest.mark.parametrize("store_v_seq", [False, True])
def test_lif_forward_op(K, recompute, store_v_seq):
    x = seeded_randn((6, 64), 1, 0.5, 1.0).cuda().requires_grad_()
    v0 = torch.zeros(64, device="cuda", requires_grad=True)
    torch.library.opcheck(K.hip_multistep_lif_forward,
                          (x, v0, 1.0, 0.0, False, False, 2.0, True, 1, 2.0, store_v_seq, 0, recompute), test_utils=TESTS)


def test_if_and_plif_forward_ops(K):
    x = seeded_randn((5, 32), 2, 0.5, 1.0).cuda().requires_grad_()
    v0 = torch.zeros(32, device="cuda")
    torch.library.opcheck(K.hip_multistep_if_forward, (x, v0, 1.0, 0.0, True, False, 0, 4.0, True, 0, True),
                          test_utils=TESTS)
    k = torch.tensor(0.5, device="cuda", requires_grad=True)
    torch.library.opcheck(K.hip_multistep_plif_forward, (x, v0, k, 1.0, 0.0, False, False, True, 1, 2.0, True, 0, True),
                          test_utils=TESTS)


@pytest.mark.parametrize("recompute", [False, True])
def test_qif_and_ilif_forward_ops(K, recompute):
    x = seeded_randn((5, 32), 6, 0.5, 0.6).cuda().requires_grad_()
    v0 = torch.zeros(32, device="cuda", requires_grad=True)
    torch.library.opcheck(K.hip_multistep_qif_forward,
                          (x, v0, 1.0, -0.1, False, False, 2.0, 0.0, 0.8, 1.0, 1, 2.0, True, 0, recompute), test_utils=TESTS)
    torch.library.opcheck(K.hip_multistep_ilif_forward, (x, v0, 1.6, 0.7, 4, 0.0, 4.0, False, True, 0, recompute),
                          test_utils=TESTS)
    torch.library.opcheck(K.hip_multistep_ilif_inference, (x.detach(), v0.detach(), 1.6, 0.7, 4, False, 0),
                          test_utils=("test_schema", "test_faketensor"))


def test_inference_and_packed_ops(K):
    x = seeded_randn((4, 48), 3, 0.5, 1.0).cuda()
    v0 = torch.zeros(48, device="cuda")
    torch.library.opcheck(K.hip_multistep_lif_inference, (x, v0, 1.0, 0.0, False, 2.0, True, True, 0),
                          test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(K.hip_multistep_lif_inference_packed, (x, v0, 1.0, 0.0, False, 2.0, True, False, 0),
                          test_utils=("test_schema", "test_faketensor"))
    torch.library.opcheck(K.hip_multistep_if_inference_packed, (x, v0, 1.0, 0.0, True, True, 0),
                          test_utils=("test_schema", "test_faketensor"))


def test_stbif_op():
    from spikingjelly_amd.activation_based.hip_kernel.stbif_kernel import hip_multistep_stbif

    x = seeded_randn((5, 40), 7, 0.0, 0.5).cuda()
    q, acc = torch.full((40,), 0.5, device="cuda"), torch.zeros(40, device="cuda")
    th = [torch.tensor(v, device="cuda") for v in (0.25, 3.0, -4.0)]
    torch.library.opcheck(hip_multistep_stbif, (x, q, acc, *th, 0), test_utils=("test_schema", "test_faketensor"))


def test_izhikevich_op():
    from spikingjelly_amd.activation_based.hip_kernel.izhikevich_kernel import hip_multistep_izhikevich_forward

    x = seeded_randn((5, 32), 9, 0.4, 0.5).cuda().requires_grad_()
    v0 = torch.zeros(32, device="cuda", requires_grad=True)
    w0 = torch.zeros(32, device="cuda", requires_grad=True)
    scalars = [2.0, 1.0, 0.0, -0.1, 0.8, 1.0, 3.0, 0.3, 0.2]
    for store in (False, True):
        torch.library.opcheck(hip_multistep_izhikevich_forward, (x, v0, w0, scalars, False, False, 1, 2.0, store, store, True, 0),
                              test_utils=TESTS)
        torch.library.opcheck(hip_multistep_izhikevich_forward,
                              (x, v0, w0, scalars, False, False, 1, 2.0, store, store, False, 0, True), test_utils=TESTS)


def test_activation_aware_if_op():
    from spikingjelly_amd.activation_based.hip_kernel.aaif_kernel import hip_multistep_activation_aware_if

    x = seeded_randn((5, 48), 8, 0.3, 0.6).cuda()
    v0 = torch.zeros(48, device="cuda")
    th, off = torch.tensor([1.0, 1.5, 2.0], device="cuda"), torch.tensor(0.25, device="cuda")
    for store in (False, True):
        torch.library.opcheck(hip_multistep_activation_aware_if, (x, v0, th, off, 3, 4, 0.0, True, store, 0),
                              test_utils=("test_schema", "test_faketensor"))


def test_ssa_op():
    from spikingjelly_amd.activation_based.hip_kernel.attention_kernel import hip_ssa_forward

    qkv = (torch.rand((2, 3, 2, 32, 20), generator=torch.Generator().manual_seed(4)) < 0.3).float().cuda().requires_grad_()
    torch.library.opcheck(hip_ssa_forward, (qkv, 0.125), test_utils=TESTS)


def test_module_traces_under_torch_compile_with_the_eager_backend():
    """The node's forward is one opaque operator to the tracer: compiling with backend='eager' must give
    the eager result (no graph breaks inside the op)."""
    from spikingjelly_amd.activation_based import functional, neuron, surrogate

    node = neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(), step_mode="m", backend="hip").cuda()
    x = seeded_randn((4, 8, 16), 5, 0.5, 1.0).cuda()
    eager = node(x)
    functional.reset_net(node)

    fn = torch.compile(lambda t: functional.lif_multi_step_hip(t, torch.zeros_like(t[0]), 2.0, True, 1.0, 0.0,
                                                               surrogate.ATan(), False, False)[0], backend="eager")
    assert torch.equal(fn(x), eager)


def _chain_inputs(T=3, B=2, Cin=8, Cout=12, Lp=8):
    x = seeded_randn((T, B, Cin, Lp), 31, 0.0, 1.5).cuda().requires_grad_()
    w = (seeded_randn((Cout, Cin), 32, 0.0, 0.4)).cuda().requires_grad_()
    gamma = seeded_randn((Cout,), 33, 1.5, 0.2).cuda().requires_grad_()
    beta = seeded_randn((Cout,), 34, 0.5, 0.3).cuda().requires_grad_()
    v0 = torch.zeros((1,), device="cuda").expand(B, Cout, Lp)
    rm, rv = torch.zeros(Cout, device="cuda"), torch.ones(Cout, device="cuda")
    tracked = torch.zeros((), dtype=torch.int64, device="cuda")
    return x, w, gamma, beta, v0, rm, rv, tracked


def test_fused_chain_ops():
    """The operators a tracing compiler sees in place of the fused convolution / batch norm / LIF chains
    (``hip_kernel/fused_ops.py``): schema (including the mutated running statistics), fake kernels, autograd
    registration and AOT dispatch."""
    from spikingjelly_amd.activation_based.hip_kernel import conv_bn_lif as C
    from spikingjelly_amd.activation_based.hip_kernel import fused_ops as O
    from spikingjelly_amd.activation_based.hip_kernel import library as L
    from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K

    flags = K._flags(False, True, True, 0)
    spec = (2.0, 1.0, 0.0, flags, 0, 4.0)
    x, w, gamma, beta, v0, rm, rv, tracked = _chain_inputs()
    terms = C._terms()
    for heads, cph in ((0, 0), (2, 2)):
        torch.library.opcheck(O.hip_conv_bn_lif_forward,
                              (x, w, gamma, beta, v0, rm, rv, True, 0.1, 1e-5, *spec, False, terms, heads, cph, 0.125),
                              test_utils=TESTS)
    y = seeded_randn((3, 2, 12, 8), 35, 0.4, 1.5).cuda().requires_grad_()
    torch.library.opcheck(O.hip_bn_lif_forward, (y, gamma, beta, v0, rm, rv, True, 0.1, 1e-5, *spec), test_utils=TESTS)
    torch.library.opcheck(O.hip_bn_lif_forward, (y, None, None, v0, rm, rv, False, 0.1, 1e-5, *spec), test_utils=TESTS)
    assert float(rm.abs().max()) == 0.0 and float((rv - 1).abs().max()) == 0.0   # the operators write to no argument
    pre = seeded_randn((3, 2, 8, 8), 36, 0.6, 1.0).cuda().requires_grad_()
    pre_v0 = torch.zeros((2, 8, 8), device="cuda")
    torch.library.opcheck(O.hip_lif_conv_bn_lif_forward,
                          (pre, pre_v0, w, gamma, beta, v0, rm, rv, True, 0.1, 1e-5, *spec, *spec, terms), test_utils=TESTS)
    # the same chains ending in a parametric LIF: k = sigmoid(w) as one more (differentiable) tensor argument
    k = torch.tensor([0.4], device="cuda", requires_grad=True)
    plif = (0.0, *spec[1:])
    torch.library.opcheck(O.hip_bn_lif_forward, (y, gamma, beta, v0, rm, rv, True, 0.1, 1e-5, *plif, k), test_utils=TESTS)
    for heads, cph in ((0, 0), (2, 2)):
        torch.library.opcheck(O.hip_conv_bn_lif_forward,
                              (x, w, gamma, beta, v0, rm, rv, True, 0.1, 1e-5, *plif, False, terms, heads, cph, 0.125, k),
                              test_utils=TESTS)
    torch.library.opcheck(O.hip_lif_conv_bn_lif_forward,
                          (pre, pre_v0, w, gamma, beta, v0, rm, rv, True, 0.1, 1e-5, *spec, *plif, terms, k), test_utils=TESTS)
    x2 = seeded_randn((3, 2 * 3 * 2 * 2 * 8), 37, 0.6, 1.0).cuda().requires_grad_()   # B = 2, 3 x 2 heads x 2 channels x 8 tokens
    torch.library.opcheck(O.hip_lif_ssa_forward, (x2, torch.zeros(x2.shape[1], device="cuda"), *spec, 6, 2, 2, 8, 0.125),
                          test_utils=TESTS)
