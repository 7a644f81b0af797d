"""HIP graph capture of a whole training step through the hip backend.

The operators launch on the current stream, never synchronise the host and allocate through torch only, so a
forward + backward step can be captured once and replayed; for small layers that removes the per-launch host cost.
Every replay is checked against the eager result, with eager work and synchronisation between replays.
"""

import pytest
import torch

from spikingjelly_amd.activation_based import functional, neuron, surrogate

from helpers import bits_equal, seeded_randn

pytestmark = pytest.mark.gpu


def _eager_step(node, x, gs):
    xi = x.clone().requires_grad_()
    s = node(xi)
    (s * gs).sum().backward()
    functional.reset_net(node)
    return s.detach().clone(), xi.grad.clone()


@pytest.mark.parametrize("cls,kw", [
    (neuron.IFNode, {}),
    (neuron.LIFNode, {"tau": 2.0}),
    (neuron.ParametricLIFNode, {"init_tau": 2.0}),
    (neuron.QIFNode, {"tau": 2.0}),
    (neuron.EIFNode, {"tau": 2.0}),
    (neuron.IzhikevichNode, {"tau": 2.0, "a": 0.3, "b": 0.2}),
    (neuron.ILIFNode, {"surrogate_function": surrogate.MultiLevelSpikeCount(4)}),
])
def test_training_step_replays_from_a_graph(cls, kw):
    kw = {"surrogate_function": surrogate.ATan(), **kw}
    node = cls(step_mode="m", backend="hip", **kw).cuda()
    T, B, C = 4, 64, 128
    static_x = seeded_randn((T, B, C), 1, 0.5, 1.0).cuda().requires_grad_()
    static_gs = seeded_randn((T, B, C), 2).cuda()

    # warm-up on a side stream, as torch's capture protocol asks
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            s = node(static_x)
            (s * static_gs).sum().backward()
            static_x.grad = None
            for p in node.parameters():
                p.grad = None
            functional.reset_net(node)
    torch.cuda.current_stream().wait_stream(side)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_s = node(static_x)
        (static_s * static_gs).sum().backward()
        functional.reset_net(node)
    static_gx = static_x.grad

    for i in range(4):
        x = seeded_randn((T, B, C), 10 + i, 0.5, 1.0).cuda()
        gs = seeded_randn((T, B, C), 20 + i).cuda()
        want_s, want_gx = _eager_step(node, x, gs)  # eager work between the replays
        torch.cuda.synchronize()
        with torch.no_grad():
            static_x.copy_(x)
            static_gs.copy_(gs)
        graph.replay()
        torch.cuda.synchronize()
        assert bits_equal(static_s.detach(), want_s), f"replay {i}: spikes"
        assert bits_equal(static_gx, want_gx), f"replay {i}: grad_x"


def test_inference_with_packed_spikes_replays_from_a_graph():
    T, N = 8, 4096
    static_x = seeded_randn((T, N), 3, 0.5, 1.0).half().cuda()
    v0 = torch.zeros(N, dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            functional.lif_multi_step_hip_packed(static_x, v0, 2.0, True, 1.0, 0.0)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_bits, static_v, _ = functional.lif_multi_step_hip_packed(static_x, v0, 2.0, True, 1.0, 0.0)
    for i in range(3):
        x = seeded_randn((T, N), 30 + i, 0.5, 1.0).half().cuda()
        want_bits, want_v, _ = functional.lif_multi_step_hip_packed(x, v0, 2.0, True, 1.0, 0.0)
        torch.cuda.synchronize()
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_bits, want_bits) and bits_equal(static_v, want_v), f"replay {i}"


def test_self_attention_block_with_packed_spikes_replays_from_a_graph():
    """The fused LIF -> contraction step (bit-packed spikes in between) inside a captured training step of the block."""
    from spikingjelly_amd.activation_based import layer

    torch.manual_seed(3)
    block = layer.SpikingSelfAttention(128, 4, backend="hip").cuda()
    with torch.no_grad():
        block.qkv_conv_bn[1].weight.fill_(2.0)
        block.proj_conv_bn[1].weight.fill_(3.0)
    for m in block.modules():  # keep the running statistics out of the comparison
        if isinstance(m, torch.nn.BatchNorm1d):
            m.momentum = 0.0
    shape = (4, 8, 128, 96)
    static_x = seeded_randn(shape, 1).cuda().requires_grad_()
    static_g = seeded_randn(shape, 2).cuda()

    def step(x, g):
        y = block(x)
        y.backward(g)
        functional.reset_net(block)
        return y

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(static_x, static_g)
            static_x.grad = None
            block.zero_grad(set_to_none=True)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = step(static_x, static_g)
    static_gx = static_x.grad
    for i in range(3):
        x, g = seeded_randn(shape, 10 + i).cuda(), seeded_randn(shape, 20 + i).cuda()
        xi = x.clone().requires_grad_()
        want = step(xi, g).detach().clone()
        want_gx = xi.grad.clone()
        block.zero_grad(set_to_none=True)
        torch.cuda.synchronize()
        with torch.no_grad():
            static_x.copy_(x)
            static_g.copy_(g)
        graph.replay()
        torch.cuda.synchronize()
        assert bits_equal(static_y.detach(), want) and float(want.mean()) > 0.02, f"replay {i}: output"
        assert bits_equal(static_gx, want_gx), f"replay {i}: grad_x"


@pytest.mark.parametrize("cls,kw", [
    (neuron.IFNode, {}),
    (neuron.LIFNode, {"tau": 2.0}),
    (neuron.ParametricLIFNode, {"init_tau": 2.0}),
])
def test_loop_of_single_steps_replays_from_a_graph(cls, kw):
    """A Python loop over time with ``step_mode='s'`` (state and its gradient carried between the calls), recorded with
    its backward by the package's helper; a replay costs one launch of the graph instead of 2 T operator calls."""
    from spikingjelly_amd.activation_based.hip_kernel.graph import GraphedStep

    node = cls(step_mode="s", backend="hip", surrogate_function=surrogate.ATan(), **kw).cuda()
    reference = cls(step_mode="m", backend="hip", surrogate_function=surrogate.ATan(), **kw).cuda()
    T, B, C = 6, 32, 96

    def step(x_seq, gs_seq):
        spikes = torch.stack([node(x_seq[t]) for t in range(x_seq.shape[0])])
        (spikes * gs_seq).sum().backward()
        functional.reset_net(node)
        return spikes.detach()

    x0 = seeded_randn((T, B, C), 1, 0.5, 1.0).cuda().requires_grad_()
    graphed = GraphedStep(step, [x0, seeded_randn((T, B, C), 2).cuda()], parameters=node.parameters())
    for i in range(4):
        x, gs = seeded_randn((T, B, C), 10 + i, 0.5, 1.0).cuda(), seeded_randn((T, B, C), 20 + i).cuda()
        want_s, want_gx = _eager_step(reference, x, gs)  # the multi-step kernels, eagerly, between the replays
        want_gw = [p.grad.clone() for p in reference.parameters()]
        reference.zero_grad(set_to_none=True)
        torch.cuda.synchronize()
        got_s = graphed(x, gs)
        torch.cuda.synchronize()
        assert bits_equal(got_s, want_s), f"replay {i}: spikes"
        assert torch.allclose(graphed.static_inputs[0].grad, want_gx, rtol=1e-5, atol=1e-6), f"replay {i}: grad_x"
        for p, w in zip(node.parameters(), want_gw):
            assert torch.allclose(p.grad, w, rtol=1e-4, atol=1e-5), f"replay {i}: parameter gradient"


def test_graphed_step_checks_what_it_is_given():
    from spikingjelly_amd.activation_based.hip_kernel.graph import GraphedStep

    x = seeded_randn((4, 64), 1).cuda()
    graphed = GraphedStep(lambda a: functional.lif_multi_step_hip(a, torch.zeros_like(a[0]), 2.0, True, 1.0, 0.0,
                                                                  surrogate.ATan())[0], [x])
    with pytest.raises(ValueError, match="recorded with"):
        graphed(x[:2])
    with pytest.raises(ValueError, match="recorded with"):
        graphed(x, x)
    with pytest.raises(ValueError, match="on the GPU"):
        GraphedStep(lambda a: a, [torch.zeros(3)])
