"""Input-compressed gradient checkpointing (``memopt/checkpointing.py``): the consumer of the spike compressors.

The CPU tests restate what the reference's own tests check for these classes
(``test/activation_based/test_checkpointing.py:160-177, 231-272, 1154-1377``) and add what pins the mechanism:
a checkpointed segment must return the outputs, states and gradients of the plain segment, must keep its input only in
compressed form, and must replay the forward's random numbers.  The GPU tests run the same comparisons with the hip
backend neurons and the HIP bit-packing kernels underneath.
"""

import copy
import logging
import pickle

import pytest
import torch
import torch.nn as nn

from spikingjelly_amd.activation_based import base, functional, neuron, surrogate
from spikingjelly_amd.activation_based.memopt import (BitSpikeCompressor, BooleanSpikeCompressor, GCContainer,
                                                      NullSpikeCompressor, TCGCContainer, Uint8SpikeCompressor,
                                                      in_gc_1st_forward, input_compressed_gc, query_autocast,
                                                      to_gc_function)
from spikingjelly_amd.activation_based.memopt import checkpointing as ckpt

from helpers import bits_equal, seeded_randn


def _linear(x, weight, bias=None):
    y = torch.matmul(x, weight.t())
    return y if bias is None else y + bias


def test_first_forward_flag_is_thread_local_and_nests():
    assert not in_gc_1st_forward()
    with ckpt._gc_1st_forward():
        assert in_gc_1st_forward()
        with ckpt._gc_1st_forward():
            assert in_gc_1st_forward()
        assert in_gc_1st_forward()
    assert not in_gc_1st_forward()
    seen = []
    input_compressed_gc(lambda x: seen.append(in_gc_1st_forward()) or x * 2, NullSpikeCompressor(),
                        torch.ones(3, requires_grad=True)).sum().backward()
    assert seen == [True, False]  # first forward, then the recomputation inside the backward


def test_autocast_query():
    device_type, dtype, enabled = query_autocast()
    assert device_type == "cpu" and dtype is not None and not enabled
    with torch.amp.autocast("cpu", dtype=torch.bfloat16):
        assert query_autocast() == ("cpu", torch.bfloat16, True)


def test_argument_separation_round_trip():
    a, b = torch.randn(3, 4), torch.randn(2, 5)
    plain, tensors, positions = ckpt._separate_args(a, "text", b, 3)
    assert plain == [None, "text", None, 3] and positions == [0, 2] and tensors[0] is a and tensors[1] is b
    combined = ckpt._combine_args(plain, tensors, positions)
    assert combined[0] is a and combined[1] == "text" and combined[2] is b and combined[3] == 3


def test_function_returns_the_plain_results_and_gradients():
    x, w, b = seeded_randn((5, 3), 1), seeded_randn((4, 3), 2), seeded_randn((4,), 3)
    with torch.no_grad():
        y = input_compressed_gc(_linear, NullSpikeCompressor(), x, w)
        assert bits_equal(y, _linear(x, w)) and not y.requires_grad
    xs = [t.clone().requires_grad_() for t in (x, w, b)]
    ys = [t.clone().requires_grad_() for t in (x, w, b)]
    out = input_compressed_gc(_linear, NullSpikeCompressor(), *xs)
    assert out.requires_grad and bits_equal(out.detach(), _linear(*ys).detach())
    g = seeded_randn(out.shape, 4)
    out.backward(g)
    _linear(*ys).backward(g)
    for got, want in zip(xs, ys):
        assert bits_equal(got.grad, want.grad)
    # an argument that does not ask for a gradient gets none and does not stop the others
    frozen = w.clone()
    x2 = x.clone().requires_grad_()
    input_compressed_gc(_linear, NullSpikeCompressor(), x2, frozen).sum().backward()
    assert x2.grad is not None and frozen.grad is None


def test_decorator_and_converter_forms():
    comp = NullSpikeCompressor()

    @to_gc_function(comp)
    def decorated(x, weight):
        """doc kept"""
        return _linear(x, weight)

    x, w = seeded_randn((5, 3), 5).requires_grad_(), seeded_randn((4, 3), 6).requires_grad_()
    assert decorated.__doc__ == "doc kept"
    assert bits_equal(decorated(x, w).detach(), _linear(x, w).detach()) and decorated(x, w).requires_grad
    converted = to_gc_function(comp, _linear)
    assert bits_equal(converted(x, w).detach(), _linear(x, w).detach())


class _Recording(NullSpikeCompressor):
    def __init__(self, inner):
        self.inner, self.kept = inner, []

    def _compress(self, s_seq):
        out = self.inner._compress(s_seq)
        self.kept.append(out)
        return out

    def _decompress(self, s_seq, shape):
        return self.inner._decompress(s_seq, shape)


@pytest.mark.parametrize("make,bytes_per_spike", [(NullSpikeCompressor, 4.0), (BooleanSpikeCompressor, 1.0),
                                                  (Uint8SpikeCompressor, 1.0), (BitSpikeCompressor, 0.125)])
def test_only_the_compressed_input_is_kept(make, bytes_per_spike):
    spikes = (seeded_randn((8, 4, 16), 7) > 0.3).float().requires_grad_()
    w = seeded_randn((6, 16), 8).requires_grad_()
    comp = _Recording(make())
    saved = []
    with torch.autograd.graph.saved_tensors_hooks(lambda t: saved.append(t) or t, lambda t: t):
        out = input_compressed_gc(_linear, comp, spikes, w)
    # what autograd holds for this segment: the compressed spikes and the weight, nothing from inside the segment
    assert len(saved) == 2 and saved[0] is comp.kept[0] and saved[1] is w
    assert saved[0].numel() * saved[0].element_size() == spikes.numel() * bytes_per_spike
    ref_s, ref_w = spikes.detach().clone().requires_grad_(), w.detach().clone().requires_grad_()
    g = seeded_randn(out.shape, 9)
    out.backward(g)
    _linear(ref_s, ref_w).backward(g)
    assert bits_equal(spikes.grad, ref_s.grad) and bits_equal(w.grad, ref_w.grad)


def test_random_numbers_of_the_forward_are_replayed():
    drop = nn.Dropout(0.5)
    x = torch.ones(4096, requires_grad=True)
    torch.manual_seed(11)
    y = input_compressed_gc(drop, NullSpikeCompressor(), x)
    after = torch.rand(1)
    y.sum().backward()
    assert bits_equal(x.grad, y.detach())  # the mask of the recomputation is the mask of the forward (both scale by 2)
    torch.manual_seed(11)
    drop(torch.ones(4096))
    assert bits_equal(after, torch.rand(1))  # and the checkpoint consumed the generator exactly once


def _snn(backend="torch", **kw):
    return [nn.Linear(12, 16), neuron.LIFNode(tau=2.0, step_mode="m", backend=backend, surrogate_function=surrogate.ATan(), **kw),
            nn.Linear(16, 8), neuron.IFNode(step_mode="m", backend=backend, surrogate_function=surrogate.Sigmoid(), **kw)]


def _run(net, x, g):
    x = x.clone().requires_grad_()
    out = net(x)
    out.backward(g)
    states = [s.detach().clone() for s in base.extract_memories(net)]
    grads = [p.grad.clone() for p in net.parameters()]
    return out.detach(), x.grad, states, grads


def test_container_basics():
    l1, l2 = nn.Linear(10, 20), nn.ReLU()
    box = GCContainer(NullSpikeCompressor(), l1, l2)
    x = seeded_randn((3, 10), 12).requires_grad_()
    assert len(box) == 2 and box[0] is l1 and box[1] is l2 and box.num_states == 0
    assert bits_equal(box(x).detach(), l2(l1(x)).detach()) and box(x).requires_grad
    assert "x_compressor=NullSpikeCompressor" in box.extra_repr()
    assert isinstance(GCContainer(None, l1).x_compressor, NullSpikeCompressor)
    stateful = GCContainer(None, neuron.IFNode(step_mode="m"))
    assert stateful.num_states == 1 and stateful(x).shape == x.shape


@pytest.mark.parametrize("make", [NullSpikeCompressor, BitSpikeCompressor])
def test_stateful_container_equals_the_plain_network(make):
    torch.manual_seed(13)
    layers = _snn()
    plain, boxed = nn.Sequential(*copy.deepcopy(layers)), GCContainer(make(), *copy.deepcopy(layers))
    x = (seeded_randn((6, 3, 12), 14) > 0.0).float()
    g = seeded_randn((6, 3, 8), 15)
    want, got = _run(plain, x, g), _run(boxed, x, g)
    assert bits_equal(got[0], want[0]) and float(want[0].mean()) > 0.02
    torch.testing.assert_close(got[1], want[1], rtol=1e-6, atol=1e-7)
    for a, b in zip(got[2] + got[3], want[2] + want[3]):
        torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-7)
    # the memories were written back: a second call continues from them, a reset returns to the sentinel
    second_plain, second_boxed = plain(x), boxed(x)
    assert bits_equal(second_boxed.detach(), second_plain.detach())
    functional.reset_net(boxed)
    assert all(not torch.is_tensor(s) for s in base.extract_memories(boxed))


@pytest.mark.parametrize("stateful", [False, True])
def test_first_segment_of_a_network_still_trains_its_parameters(stateful):
    """Data that requires no gradient into a checkpointed segment: its parameters must get the gradients of the plain
    segment (the segment's arguments carry no graph then; an anchor argument keeps the function in the graph)."""
    torch.manual_seed(31)
    layers = _snn()[:2] if stateful else [nn.Linear(12, 16), nn.ReLU()]
    plain, boxed = nn.Sequential(*copy.deepcopy(layers)), GCContainer(BitSpikeCompressor(), *copy.deepcopy(layers))
    x = (seeded_randn((6, 3, 12), 32) > 0.0).float()
    g = seeded_randn((6, 3, 16), 33)
    for net in (plain, boxed):
        out = net(x)
        assert out.requires_grad
        out.backward(g)
    for a, b in zip(boxed.parameters(), plain.parameters()):
        assert a.grad is not None
        torch.testing.assert_close(a.grad, b.grad, rtol=1e-6, atol=1e-7)
    with torch.no_grad():  # and without a graph nothing is anchored
        assert not boxed(x).requires_grad


def test_container_survives_deepcopy_and_pickle():
    box = GCContainer(None, neuron.IFNode(step_mode="m"))
    x = torch.rand(4, 2, 3, generator=torch.Generator().manual_seed(16))
    with torch.no_grad():
        want = box(x)
    functional.reset_net(box)
    copied, restored = copy.deepcopy(box), pickle.loads(pickle.dumps(box))
    assert copied.f_forward is not box.f_forward
    with torch.no_grad():
        assert bits_equal(copied(x), want) and bits_equal(restored(x), want)
    assert not torch.is_tensor(box[0].v)  # the copies ran on their own memories


def test_temporal_chunks_equal_the_whole_sequence():
    torch.manual_seed(17)
    layers = _snn()
    whole, chunked = GCContainer(None, *copy.deepcopy(layers)), TCGCContainer(None, *copy.deepcopy(layers), n_chunk=3)
    x = (seeded_randn((8, 3, 12), 18) > 0.0).float()
    g = seeded_randn((8, 3, 8), 19)
    want, got = _run(whole, x, g), _run(chunked, x, g)
    assert bits_equal(got[0], want[0])
    for a, b in zip([got[1]] + got[2] + got[3], [want[1]] + want[2] + want[3]):
        torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-7)
    assert "n_chunk=3" in chunked.extra_repr() and "x_compressor=NullSpikeCompressor" in chunked.extra_repr()


def test_temporal_chunk_lengths_and_cap(caplog):
    class Lengths(nn.Module):
        def __init__(self):
            super().__init__()
            self.seen = []

        def forward(self, x):
            self.seen.append(x.shape[0])
            return x

    rec = Lengths()
    x = seeded_randn((4, 2), 20)
    with torch.no_grad():
        assert bits_equal(TCGCContainer(None, rec, n_chunk=3)(x), x)
    assert rec.seen == [2, 1, 1]
    rec = Lengths()
    with caplog.at_level(logging.WARNING, logger="spikingjelly_amd"), torch.no_grad():
        assert bits_equal(TCGCContainer(None, rec, n_chunk=5)(x[:3]), x[:3])
    assert rec.seen == [1, 1, 1]
    assert "n_chunk=5" in caplog.text and "T=3" in caplog.text and "using n_chunk=3" in caplog.text
    with pytest.raises(RuntimeError), torch.no_grad():
        TCGCContainer(None, Lengths(), n_chunk=3)(torch.empty(0, 2))


def test_temporal_chunks_with_several_inputs_states_and_outputs():
    class Pair(nn.Module):
        def __init__(self):
            super().__init__()
            self.left, self.right = nn.Linear(4, 4, bias=False), nn.Linear(4, 4, bias=False)

        def forward(self, x, y):
            return self.left(x), self.right(y)

    class Running(base.MemoryModule):
        def __init__(self):
            super().__init__()
            self.register_memory("left", 0.0)
            self.register_memory("right", 0.0)
            self.step_mode = "m"

        def single_step_functional_forward(self, inputs, states, **kwargs):
            left, right = states[0] + inputs[0], states[1] + inputs[1]
            return (left, right), (left, right)

    torch.manual_seed(21)
    layers = [Pair(), Running()]
    whole = GCContainer(None, *copy.deepcopy(layers))
    chunked = TCGCContainer(None, *copy.deepcopy(layers), n_chunk=3, n_seq_inputs=2, n_outputs=2)
    x, y = seeded_randn((6, 2, 4), 22), seeded_randn((6, 2, 4), 23)
    ins_w = [t.clone().requires_grad_() for t in (x, y)]
    ins_c = [t.clone().requires_grad_() for t in (x, y)]
    out_w, out_c = whole(*ins_w), chunked(*ins_c)
    for a, b in zip(out_c, out_w):
        torch.testing.assert_close(a, b)
    for a, b in zip(base.extract_memories(chunked), base.extract_memories(whole)):
        torch.testing.assert_close(a, b)
    sum(o.sum() for o in out_w).backward()
    sum(o.sum() for o in out_c).backward()
    for a, b in zip(ins_c + list(chunked.parameters()), ins_w + list(whole.parameters())):
        torch.testing.assert_close(a.grad, b.grad)


# ---- on the GPU: hip backend neurons inside the segment, HIP bit-packing for its input -------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("chunks", [0, 2])
def test_hip_segment_with_bit_packed_input_equals_the_plain_hip_network(chunks):
    torch.manual_seed(24)
    layers = [m.cuda() for m in _snn("hip")]
    plain = nn.Sequential(*copy.deepcopy(layers))
    boxed = (TCGCContainer(BitSpikeCompressor(), *copy.deepcopy(layers), n_chunk=chunks) if chunks
             else GCContainer(BitSpikeCompressor(), *copy.deepcopy(layers)))
    x = (seeded_randn((8, 32, 12), 25) > 0.0).float().cuda()
    g = seeded_randn((8, 32, 8), 26).cuda()
    kept = []
    with torch.autograd.graph.saved_tensors_hooks(lambda t: kept.append(t) or t, lambda t: t):
        xb = x.clone().requires_grad_()
        out = boxed(xb)
    packed = [t for t in kept if t.dtype == torch.uint8]
    assert packed and all(t.is_cuda for t in packed) and sum(t.numel() for t in packed) == x.numel() // 8
    assert not any(t.shape == x.shape[: t.dim()] and t.dtype == x.dtype and t.dim() == x.dim() for t in kept)
    out.backward(g)
    want = _run(plain, x, g)
    assert bits_equal(out.detach().cpu(), want[0].cpu()) and float(want[0].mean()) > 0.005
    torch.testing.assert_close(xb.grad, want[1], rtol=1e-5, atol=1e-6)
    for a, b in zip([s.detach() for s in base.extract_memories(boxed)] + [p.grad for p in boxed.parameters()],
                    want[2] + want[3]):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_hip_segment_replays_gpu_random_numbers():
    drop = nn.Dropout(0.5)
    x = torch.ones(1 << 16, device="cuda", requires_grad=True)
    torch.manual_seed(27)
    y = input_compressed_gc(drop, NullSpikeCompressor(), x)
    y.sum().backward()
    assert bits_equal(x.grad.cpu(), y.detach().cpu())
