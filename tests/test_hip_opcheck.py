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
