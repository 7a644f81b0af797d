"""CPU-only tests of the host-side mirror of the reference interface (torch backend + plumbing):
function-vs-module consistency, memory semantics, backend validation, surrogate registry, the CPU
path of the bit compressor, operator schemas / fake kernels."""

import copy

import pytest
import torch

from oracle import neuron_oracle as no
from spikingjelly_amd.activation_based import base, functional, neuron, surrogate
from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K
from spikingjelly_amd.activation_based.hip_kernel.surrogate_registry import resolve_sg_hip_id_and_alpha
from spikingjelly_amd.activation_based.memopt import BitSpikeCompressor, BooleanSpikeCompressor

from helpers import bits_equal, seeded_randn

NODES = [
    (neuron.IFNode, {}, "if", None),
    (neuron.LIFNode, {"tau": 2.5}, "lif", 2.5),
    (neuron.LIFNode, {"tau": 5.0, "decay_input": False}, "lif", 5.0),
    (neuron.ParametricLIFNode, {"init_tau": 2.5}, "plif", None),
]


@pytest.mark.parametrize("cls,kw,kind,tau", NODES)
@pytest.mark.parametrize("v_reset", [0.0, -0.2, None])
@pytest.mark.parametrize("store_v_seq", [False, True])
def test_torch_backend_module_equals_oracle(cls, kw, kind, tau, v_reset, store_v_seq):
    x = seeded_randn((5, 3, 17), 1, 0.4, 1.0)
    gs = seeded_randn((5, 3, 17), 2)
    node = cls(v_threshold=0.7, v_reset=v_reset, surrogate_function=surrogate.ATan(), step_mode="m",
               store_v_seq=store_v_seq, **kw)
    xi = x.clone().requires_grad_()
    s = node(xi)
    s.backward(gs)
    p = node.w.detach() if kind == "plif" else tau
    ref = no.forward_backward(kind, x, torch.full((3, 17), 0.0 if v_reset is None else v_reset), gs, None, None, p,
                              kw.get("decay_input", True), 0.7, v_reset, "atan", 2.0, False)
    assert bits_equal(s.detach(), ref["spike_seq"])
    assert bits_equal(node.v.detach(), ref["v_seq"][-1])
    assert bits_equal(xi.grad, ref["grad_x"])
    if store_v_seq:
        assert bits_equal(node.v_seq.detach(), ref["v_seq"])
    else:
        assert node.v_seq is None


def test_functional_forward_is_pure():
    node = neuron.LIFNode(step_mode="m")
    x = seeded_randn((4, 2, 8), 3, 0.5, 1.0)
    (s,), (v,) = node.functional_forward((x,), (0.0,))
    assert node.v == 0.0 and isinstance(node.v, float)
    assert bits_equal(s, node(x)) and bits_equal(v, node.v)


def test_single_step_and_multi_step_agree():
    a = neuron.LIFNode(step_mode="s")
    b = neuron.LIFNode(step_mode="m")
    x = seeded_randn((6, 2, 8), 4, 0.5, 1.0)
    assert bits_equal(torch.stack([a(x[t]) for t in range(6)]), b(x))


def test_eval_mode_uses_heaviside_for_if_and_lif_only():
    x = seeded_randn((3, 4), 5, 0.5, 1.0).requires_grad_()
    lif = neuron.LIFNode(step_mode="m", surrogate_function=surrogate.ATan()).eval()
    assert not lif(x).requires_grad  # plain Heaviside: no gradient path through the spike
    plif = neuron.ParametricLIFNode(step_mode="m", surrogate_function=surrogate.ATan()).eval()
    assert plif(x).requires_grad  # PLIF keeps its surrogate in eval
    prim = neuron.LIFNode(step_mode="m", surrogate_function=surrogate.ATan(spiking=False)).eval()
    out = prim(x)
    assert ((out > 0) & (out < 1)).any()  # primitive mode stays smooth in eval


def test_memory_semantics():
    node = neuron.IFNode(step_mode="m")
    assert "v" not in node.state_dict() and dict(node.named_memories()) == {"v": 0.0}
    node(torch.ones(2, 3, 4))
    assert isinstance(node.v, torch.Tensor) and node.v.shape == (3, 4)
    node(torch.ones(2, 5, 4))  # batch size change: re-initialised, no error
    assert node.v.shape == (5, 4)
    node.reset()
    assert node.v == 0.0 and node.v_seq is None
    node.store_v_seq = True
    node(torch.ones(2, 3, 4))
    assert node.v_seq.shape == (2, 3, 4)
    node.store_v_seq = True
    assert node.v_seq is None  # setting the property clears it
    clone = copy.deepcopy(node)
    clone(torch.ones(2, 3, 4))
    assert node.v_seq is None
    with pytest.raises(AssertionError):
        node.register_memory("v_threshold", 1.0)
    hard = neuron.IFNode(v_reset=-0.5)
    assert hard.v == -0.5 and hard.get_reset_value("v") == -0.5
    x = torch.ones(3, requires_grad=True)
    hard(x)
    assert hard.v.requires_grad
    hard.detach()
    assert not hard.v.requires_grad


def test_backend_and_step_mode_validation():
    node = neuron.LIFNode()
    assert node.supported_backends == ("torch", "hip")  # both step modes have the hip backend
    with pytest.raises(NotImplementedError, match="triton is not a supported backend"):
        node.backend = "triton"
    node.step_mode = "m"
    assert node.supported_backends == ("torch", "hip")
    node.backend = "hip"
    with pytest.raises(NotImplementedError):
        node.backend = "cupy"
    with pytest.raises(ValueError):
        node.step_mode = "x"
    with pytest.raises(AssertionError):
        neuron.LIFNode(tau=1.0)
    with pytest.raises(AssertionError):
        neuron.IFNode(v_threshold=1)
    assert "backend=hip" in repr(node) and "tau=2.0" in repr(node)


def test_check_backend_library_reports_missing_library(monkeypatch):
    from spikingjelly_amd.activation_based.hip_kernel import library

    monkeypatch.setattr(library, "_lib", None)
    monkeypatch.setattr(library, "library_path", lambda: "/nonexistent/libsjhip.so")
    with pytest.raises(ImportError, match="libsjhip.so"):
        base.check_backend_library("hip")


def test_net_helpers():
    net = torch.nn.Sequential(neuron.IFNode(), torch.nn.Linear(4, 4), neuron.ParametricLIFNode())
    functional.set_step_mode(net, "m")
    assert net[0].step_mode == "m" and net[2].step_mode == "m"
    functional.set_backend(net, "hip", instance=neuron.IFNode)
    assert net[0].backend == "hip" and net[2].backend == "torch"
    net[2](torch.ones(2, 3, 4))
    functional.reset_net(net)
    functional.reset_net(net)  # cached module list path
    assert net[2].v == 0.0
    x = torch.ones(2, 3, 4, requires_grad=True)
    net[2](x)
    functional.detach_net(net)
    assert not net[2].v.requires_grad


def test_surrogate_objects_and_registry():
    assert repr(surrogate.ATan()) == "ATan(alpha=2.0, spiking=True)"
    assert resolve_sg_hip_id_and_alpha(surrogate.Sigmoid()) == (0, 4.0)
    assert resolve_sg_hip_id_and_alpha(surrogate.ATan(alpha=torch.tensor([3.0]))) == (1, 3.0)
    assert resolve_sg_hip_id_and_alpha(surrogate.Erf()) == (6, 2.0)
    with pytest.raises(NotImplementedError, match="PiecewiseLeakyReLU"):
        resolve_sg_hip_id_and_alpha(surrogate.PiecewiseLeakyReLU())
    with pytest.raises(TypeError):
        resolve_sg_hip_id_and_alpha(surrogate.ATan(alpha=torch.ones(2)))
    x = torch.tensor([-0.75, -0.25, 0.25, 0.75], dtype=torch.float64)
    for cls in (surrogate.Sigmoid, surrogate.ATan, surrogate.PiecewiseQuadratic, surrogate.PiecewiseExp,
                surrogate.SoftSign, surrogate.Erf, surrogate.PiecewiseLeakyReLU):
        f = cls()
        xs = x.clone().requires_grad_()
        out = f(xs)
        out.sum().backward()
        f.set_spiking_mode(False)
        fd = (f(x + 1e-5) - f(x - 1e-5)) / 2e-5
        assert torch.equal(out.detach(), surrogate.heaviside(x))
        torch.testing.assert_close(xs.grad, fd, atol=1e-4, rtol=1e-4)


def test_bit_compressor_cpu_path():
    spikes = torch.tensor([[1.0, 0.0, 1.0], [0.0, 1.0, 0.0]])
    c = BitSpikeCompressor()
    packed = c.compress(spikes)
    assert packed.device.type == "cpu" and packed.tolist() == [0b010101]
    torch.testing.assert_close(c.decompress(packed, tuple(spikes.shape)), spikes)
    b = BooleanSpikeCompressor()
    assert torch.equal(b.decompress(b.compress(spikes.half()), spikes.shape), spikes.half())


def test_operator_schemas_and_fake_kernels():
    """Shapes under fake tensors: (x.shape, x.shape | (0,), v.shape, x.shape), like
    test_compile_compat.py:496-525 checks for the reference ops."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    assert "Tensor? grad_v_seq" in str(torch.ops.sj.hip_multistep_lif_backward.default._schema)
    with FakeTensorMode():
        x = torch.empty(5, 12)
        v = torch.empty(12)
        s, v_seq, v_last, h = torch.ops.sj.hip_multistep_lif_forward(x, v, 1.0, 0.0, False, False, 2.0, True, 1, 2.0,
                                                                     True, 0, False)
        assert s.shape == v_seq.shape == h.shape == (5, 12) and v_last.shape == (12,)
        _, _, _, h = torch.ops.sj.hip_multistep_lif_forward(x, v, 1.0, 0.0, False, False, 2.0, True, 1, 2.0, True, 0,
                                                            True)
        assert h.shape == (0,)  # replay path keeps no h_seq
        s, v_seq, v_last = torch.ops.sj.hip_multistep_if_inference(x, v, 1.0, 0.0, True, False, 0)
        assert v_seq.shape == (0,) and v_last.shape == (12,)
        gx, gvi, gk = torch.ops.sj.hip_multistep_plif_backward(x, None, None, None, x, v, torch.empty(()), 1.0, 0.0,
                                                               False, False, True, 0, 4.0, 0)
        assert gx.shape == (5, 12) and gvi.shape == (12,) and gk.shape == ()


def test_functional_names_follow_the_backend_naming_rule():
    """<neuron>_multi_step_<backend>, fully annotated, exported (reference
    test/activation_based/test_functional_neuron.py:709-732)."""
    import inspect

    for name in ("if_multi_step_hip", "lif_multi_step_hip", "plif_multi_step_hip"):
        fn = getattr(functional, name)
        sig = inspect.signature(fn)
        assert all(p.annotation is not inspect.Parameter.empty for p in sig.parameters.values())
        assert sig.return_annotation is not inspect.Signature.empty
        assert list(sig.parameters)[-2:] == ["detach_reset", "store_v_seq"]


def test_hip_bit_packing_refuses_cpu_tensors():
    """The device functions have no other path: a CPU tensor raises instead of being packed by torch ops."""
    from spikingjelly_amd.activation_based.hip_kernel import compress as hip_compress

    with pytest.raises(RuntimeError, match="ROCm device"):
        hip_compress.bit_spike_compress(torch.ones(16))
    with pytest.raises(RuntimeError, match="ROCm device"):
        hip_compress.bit_spike_decompress(torch.zeros(2, dtype=torch.uint8), (16,))


# ---- tree-wide memory helpers (reference base.py:1128-1551; cases follow test/activation_based/test_memory.py) ----
class _Counter(base.MemoryModule):
    """Stateful in the classic style: the forward reads and writes its own memories."""

    def __init__(self, start=0.0):
        super().__init__()
        self.register_memory("count", torch.tensor(start))
        self.register_memory("total", torch.tensor(0.0))

    def single_step_forward(self, x, *, scale=1.0):
        self.count = self.count + 1.0
        self.total = self.total + x.sum() * scale
        return x * self.count


def _memory_tree():
    net = torch.nn.Sequential(_Counter(), torch.nn.Identity(), torch.nn.Sequential(_Counter(5.0)))
    return net


def test_named_memories_walks_the_tree_in_registration_order():
    net = _memory_tree()
    names = [n for n, _ in base.named_memories(net)]
    assert names == ["0.count", "0.total", "2.0.count", "2.0.total"]
    assert [n for n, _ in base.named_memories(net, prefix="net")] == ["net." + n for n in names]
    assert [float(v) for v in base.memories(net)] == [0.0, 0.0, 5.0, 0.0]
    assert list(base.named_memories(torch.nn.Linear(2, 2))) == []


def test_extract_and_load_memories_round_trip_and_length_check():
    net = _memory_tree()
    net(torch.ones(3))
    taken = base.extract_memories(net)
    assert [float(v) for v in taken] == [1.0, 3.0, 6.0, 3.0]
    base.load_memories(net, [v + 10 for v in taken])
    assert [float(v) for v in base.extract_memories(net)] == [11.0, 13.0, 16.0, 13.0]
    assert float(net[2][0].count) == 16.0
    with pytest.raises(ValueError, match="mismatch"):
        base.load_memories(net, taken[:-1])
    with pytest.raises(ValueError, match="mismatch"):
        base.load_memories(net, taken + [torch.tensor(0.0)])
    assert [float(v) for v in base.extract_memories(net)] == [11.0, 13.0, 16.0, 13.0]  # nothing half-written


def test_to_functional_forward_swaps_states_in_and_restores_them():
    module = _Counter(7.0)
    f = base.to_functional_forward(module)
    x = torch.tensor([1.0, 2.0])
    outputs, states = f((x,), (torch.tensor(1.0), torch.tensor(4.0)), scale=2.0)
    assert torch.equal(outputs[0], x * 2.0)
    assert [float(s) for s in states] == [2.0, 10.0]
    assert float(module.count) == 7.0 and float(module.total) == 0.0
    with pytest.raises(ValueError, match="expected 2 states"):
        f((x,), (torch.tensor(1.0),))

    class Failing(_Counter):
        def single_step_forward(self, x):
            self.count = self.count + x
            raise RuntimeError("expected failure")

    bad = Failing(3.0)
    with pytest.raises(RuntimeError, match="expected failure"):
        base.to_functional_forward(bad)((torch.tensor(1.0),), (torch.tensor(0.0), torch.tensor(0.0)))
    assert float(bad.count) == 3.0


def test_to_functional_forward_nested_stateless_and_custom_fn():
    net = _memory_tree()
    f = base.to_functional_forward(net)
    x = torch.ones(2)
    start = tuple(torch.tensor(v) for v in (1.0, 0.0, 2.0, 0.0))
    outputs, states = f((x,), start)
    assert torch.equal(outputs[0], x * 2.0 * 3.0)
    assert [float(s) for s in states] == [2.0, 2.0, 3.0, 4.0]
    assert [float(v) for v in base.extract_memories(net)] == [0.0, 0.0, 5.0, 0.0]

    lin = torch.nn.Linear(4, 2)
    outputs, states = base.to_functional_forward(lin)((torch.ones(3, 4),), ())
    assert states == () and torch.equal(outputs[0], lin(torch.ones(3, 4)))

    module = _Counter()
    outputs, states = base.to_functional_forward(module, lambda x: (x + module.count, x))(
        (torch.tensor(1.0),), (torch.tensor(4.0), torch.tensor(0.0)))
    assert [float(o) for o in outputs] == [5.0, 1.0] and float(states[0]) == 4.0


def test_to_functional_forward_uses_pure_forwards_without_touching_memories():
    class Pure(base.MemoryModule):
        def __init__(self):
            super().__init__()
            self.register_memory("left", torch.tensor(10.0))
            self.register_memory("right", torch.tensor(20.0))

        def single_step_functional_forward(self, inputs, states, **kwargs):
            left, right = states[0] + inputs[0], states[1] + inputs[1]
            return (left, right), (left, right)

        def forward(self, *args, **kwargs):
            raise AssertionError("the stateful path was used")

    class Split(torch.nn.Module):
        def forward(self, x, y, *, scale=1.0):
            return (x + y) * scale, x - y

    pure = Pure()
    outputs, states = base.to_functional_forward(torch.nn.Sequential(Split(), pure))(
        (torch.tensor(3.0), torch.tensor(2.0)), (torch.tensor(1.0), torch.tensor(4.0)), scale=2.0)
    assert [float(o) for o in outputs] == [11.0, 5.0] and [float(s) for s in states] == [11.0, 5.0]
    assert float(pure.left) == 10.0 and float(pure.right) == 20.0

    # multi-step mode falls back on the default loop over single_step_functional_forward
    class Running(base.MemoryModule):
        def __init__(self):
            super().__init__()
            self.register_memory("state", torch.tensor(0.0))
            self.step_mode = "m"

        def single_step_functional_forward(self, inputs, states, **kwargs):
            state = states[0] + inputs[0]
            return (state,), (state,)

        def forward(self, *args, **kwargs):
            raise AssertionError("the stateful path was used")

    outputs, states = base.to_functional_forward(Running())((torch.tensor([1.0, 2.0, 3.0]),), (torch.tensor(4.0),))
    assert outputs[0].tolist() == [5.0, 7.0, 10.0] and float(states[0]) == 10.0

    # a sequential of stateless stages passes tuples on as positional arguments
    class Combine(torch.nn.Module):
        def forward(self, total, difference):
            return total + difference

    outputs, states = base.to_functional_forward(torch.nn.Sequential(Split(), Combine()))(
        (torch.tensor(3.0), torch.tensor(2.0)), (), scale=2.0)
    assert states == () and float(outputs[0]) == 11.0


def test_to_functional_forward_on_a_neuron_matches_the_module():
    node = neuron.LIFNode(tau=2.0, step_mode="m")
    node.v = torch.full((5,), 0.25)
    x_seq = torch.randn(6, 5, generator=torch.Generator().manual_seed(3))
    outputs, states = base.to_functional_forward(node)((x_seq,), (torch.zeros(5),))
    ref = neuron.LIFNode(tau=2.0, step_mode="m")
    assert torch.equal(outputs[0], ref(x_seq)) and torch.equal(states[0], ref.v)
    assert torch.equal(node.v, torch.full((5,), 0.25))


# ---- ILIF (reference neuron/ilif.py, test/activation_based/test_ilif_node.py:314-440) -------------------------------
def test_ilif_node_construction_and_torch_backend_known_answers():
    with pytest.raises(ValueError, match="MultiLevelSpikeCount"):
        neuron.ILIFNode(surrogate_function=surrogate.Sigmoid())
    with pytest.raises(ValueError, match="MultiLevelSpikeCount"):
        neuron.ILIFNode(surrogate_function=surrogate.MultiLevelSpikeCount(4, spiking=False))
    with pytest.raises(TypeError):
        surrogate.MultiLevelSpikeCount(2.5)
    with pytest.raises(TypeError):
        surrogate.MultiLevelSpikeCount(True)
    with pytest.raises(ValueError):
        surrogate.MultiLevelSpikeCount(0)
    with pytest.raises(ValueError):
        surrogate.MultiLevelSpikeCount(4, grad_window=(2.0, 1.0))
    node = neuron.ILIFNode()
    assert isinstance(node, neuron.LIFNode) and node.tau == pytest.approx(4.0 / 3.0)
    assert node.decay_input is False and node.v_reset is None
    assert node.surrogate_function.max_spike_count == 4
    assert (node.surrogate_function.grad_min, node.surrogate_function.grad_max) == (0.0, 4.0)
    assert node.supported_backends == ("torch", "hip")
    # non-spiking mode of the surrogate is the clamp itself
    assert torch.equal(surrogate.MultiLevelSpikeCount(4, spiking=False)(torch.tensor([-1.0, 2.5, 9.0])),
                       torch.tensor([0.0, 2.5, 4.0]))

    node = neuron.ILIFNode(v_threshold=1.0, tau=4.0 / 3.0)
    x = torch.tensor([[3.2, 0.4, 5.8]])
    y = node(x)
    assert torch.equal(y, torch.tensor([[3.0, 0.0, 4.0]]))
    torch.testing.assert_close(node.v, x - y)
    node = neuron.ILIFNode(v_threshold=1.0, tau=4.0 / 3.0)
    node(torch.tensor([[3.2]]))
    assert torch.equal(node(torch.tensor([[0.0]])), torch.tensor([[0.0]]))
    torch.testing.assert_close(node.v, torch.tensor([[0.05]]))

    # train and eval fire the same counts; multi-step equals the oracle
    kw = dict(v_threshold=0.5, tau=4.0 / 3.0, step_mode="m", store_v_seq=True)
    a, b = neuron.ILIFNode(**kw), neuron.ILIFNode(**kw).eval()
    x_seq = torch.tensor([[[1.6, -0.2]], [[0.0, 2.2]], [[0.4, 0.0]]])
    a.v = torch.tensor([[0.2, -0.1]])
    b.v = torch.tensor([[0.2, -0.1]])
    ya, yb = a(x_seq), b(x_seq)
    assert torch.equal(ya, yb) and torch.equal(a.v_seq, b.v_seq) and float(ya.max()) > 1.0
    es, ev, _ = no.multi_step("ilif", x_seq, torch.tensor([[0.2, -0.1]]), 4.0 / 3.0, False, 0.5, None,
                              no.multi_level_spike_count(4))
    assert torch.equal(ya, es) and torch.equal(a.v_seq, ev)

    with pytest.raises(ValueError, match="MultiLevelSpikeCount"):
        functional.ilif_multi_step_hip(x_seq, torch.zeros(1, 2), 2.0, 1.0, surrogate.ATan())


# ---- ST-BIF (reference neuron/spikezip.py, test_ann2snn_transformer.py:792-896, test_functional_neuron.py:690-705) ---
def test_stbif_neuron_construction_and_torch_backend():
    for bad in (1, 0, True):
        with pytest.raises(ValueError, match="level"):
            neuron.STBIFNeuron(0.25, level=bad, sym=True)
    node = neuron.STBIFNeuron(0.25, level=8, sym=True)
    assert node.supported_backends == ("torch", "hip")
    assert (float(node.pos_max), float(node.neg_min)) == (3.0, -4.0)
    assert (float(neuron.STBIFNeuron(0.5, level=8).pos_max), float(neuron.STBIFNeuron(0.5, level=8).neg_min)) == (7.0, 0.0)
    assert "q_threshold" in node.state_dict() and node.q is None and node.is_work is False
    with pytest.raises(RuntimeError, match="accumulated"):
        node.accumulated

    class Quantizer(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.s = torch.nn.Parameter(torch.tensor(0.25))
            self.sym = True
            self.pos_max, self.neg_min = torch.tensor(3), torch.tensor(-4)

    from_q = neuron.STBIFNeuron.from_quantizer(Quantizer())
    assert from_q.level == 8 and float(from_q.q_threshold) == 0.25 and not from_q.q_threshold.requires_grad

    x = torch.tensor([[-0.75, -0.2, 0.3, 0.9]])
    total = sum(node(x if t == 0 else torch.zeros_like(x)) for t in range(16))
    assert total.tolist() == [[-0.75, -0.25, 0.25, 0.75]]
    assert torch.equal(node.accumulated, total)

    # multi-step equals the loop of single steps; is_work follows inputs and outputs
    node.reset()
    assert node.q is None and node.is_work is False
    x_seq = torch.cat([x[None], torch.zeros(15, 1, 4)])
    functional.set_step_mode(node, "m")
    y_seq = node(x_seq)
    other = neuron.STBIFNeuron(0.25, level=8, sym=True)
    assert torch.equal(y_seq, torch.stack([other(v) for v in x_seq])) and node.is_work
    node.reset()
    node(torch.zeros(2, 2, 3))
    assert not node.is_work
    node(torch.stack([torch.zeros(2, 3), torch.full((2, 3), 0.25)]))
    assert node.is_work
    # a changed shape starts from fresh states
    assert node(torch.zeros(2, 5)).shape == (2, 5) and float(node.q.mean()) == 0.5


# ---- activation-aware IF (reference neuron/integrate_and_fire.py:536-1150, test_activation_aware_ifnode.py) -----------
def test_activation_aware_if_node_on_the_torch_backend():
    for kw in (dict(v_threshold=torch.ones(2, 2)), dict(v_threshold=torch.tensor([1.0, -1.0])), dict(v_offset=float("inf")),
               dict(v_reset=1), dict(channel_dim=1.0), dict(backend="cupy"), dict(detach_reset=1), dict(store_v_seq=1)):
        with pytest.raises(ValueError):
            neuron.ActivationAwareIFNode(**kw)
    node = neuron.ActivationAwareIFNode(v_threshold=torch.tensor([1.0, 2.0]), v_offset=torch.tensor([0.0, 0.5]))
    assert node.supported_backends == ("torch",) and "v_threshold" in node.state_dict()
    node.step_mode = "m"
    assert node.supported_backends == ("torch", "hip")
    with pytest.raises(ValueError, match="channels"):
        node(torch.zeros(2, 3, 5))

    # the reference tests' literal inputs (test_activation_aware_ifnode.py:253-352) against the oracle
    x = torch.tensor([[[0.8, 1.0], [1.2, 0.2]], [[0.6, 0.2], [0.4, 1.4]], [[0.3, 0.9], [0.1, 0.2]]])
    node = neuron.ActivationAwareIFNode(v_threshold=1.5, v_offset=0.25, step_mode="m")
    es, ev = no.activation_aware_if_multi_step(x, torch.zeros(2, 2), 1.5, 0.25, -1, None)
    assert torch.equal(node(x), es) and torch.equal(node.v, ev[-1])
    x = torch.tensor([[[1.1, 1.5]], [[0.2, 0.7]], [[0.8, 0.1]]])
    node = neuron.ActivationAwareIFNode(v_threshold=torch.tensor([1.0, 2.0]), v_reset=0.25, step_mode="m", store_v_seq=True)
    es, ev = no.activation_aware_if_multi_step(x, torch.full((1, 2), 0.25), torch.tensor([1.0, 2.0]), 0.0, -1, 0.25)
    assert torch.equal(node(x), es) and torch.equal(node.v_seq, ev)
    node.store_v_seq = False
    assert node.v_seq is None
    # shape change restarts from v_reset; reset restores the scalar
    node = neuron.ActivationAwareIFNode(v_threshold=1.0, v_reset=0.25)
    node(torch.tensor([[1.1]]))
    assert torch.equal(node(torch.tensor([[0.3, 0.3]])), torch.zeros(1, 2)) and torch.equal(node.v, torch.full((1, 2), 0.55))
    node.reset()
    assert node.v == 0.25
    # gradients flow on the torch backend
    node = neuron.ActivationAwareIFNode(v_threshold=torch.tensor([1.0, 2.0]), v_offset=torch.tensor([0.0, 0.25]))
    xg = torch.tensor([[0.9, 1.8]], requires_grad=True)
    node(xg).sum().backward()
    assert xg.grad is not None and bool((xg.grad != 0).all())


def test_fused_chain_steps_aside_for_hooks_and_autocast():
    """``layer.fused.unobserved``: hooks only fire through ``Module.__call__`` and autocast would change the convolution's
    dtype, so either keeps the modules of a chain in charge (reference forward: layer/attention.py:370-384)."""
    import torch.nn as nn

    from spikingjelly_amd.activation_based.layer import fused

    conv, bn, node = nn.Conv1d(4, 4, 1, bias=False), nn.BatchNorm1d(4), neuron.LIFNode(step_mode="m")
    assert fused.unobserved(conv, bn, node, None)
    for module, register in ((node, "register_forward_hook"), (conv, "register_forward_pre_hook"),
                             (bn, "register_full_backward_hook"), (conv, "register_full_backward_pre_hook")):
        handle = getattr(module, register)(lambda *a: None)
        assert not fused.unobserved(conv, bn, node)
        handle.remove()
        assert fused.unobserved(conv, bn, node)
    handle = nn.modules.module.register_module_forward_hook(lambda *a: None)
    try:
        assert not fused.unobserved(conv)
    finally:
        handle.remove()
    with torch.autocast("cpu", dtype=torch.bfloat16):
        assert fused.unobserved(conv)  # (autocast of another device type does not concern device tensors)
    assert fused.unobserved(conv, bn, node)
