"""Bool / bit spike cache (``hip_kernel/tensor_cache.py``) and the spike operators built on it (``hip_kernel/spike_op.py``).

The byte layout is pinned against ``numpy.packbits(..., bitorder="little")``, a library routine; the cache against the
reference's own literal case (17 elements, ``arange % 3 == 0``, stored twice and fetched twice at both levels,
``test/activation_based/test_cuda_custom_op_migration.py:179-190``).  The operators compute with torch's own linear and
convolution routines, so they are checked against those: same outputs and gradients, and autograd holding the
spikes only as bool or bits.
"""

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from spikingjelly_amd import configure
from spikingjelly_amd.activation_based.hip_kernel import spike_op, tensor_cache
from spikingjelly_amd.activation_based.hip_kernel.tensor_cache import (BOOL_TENSOR_CACHE, BoolTensorCache,
                                                                        bool_spike_to_float, float_spike_to_bool,
                                                                        tensor_key)

from helpers import bits_equal, seeded_randn


def _spikes(shape, seed, dtype=torch.float32):
    return (seeded_randn(shape, seed) > 0.2).to(dtype)


@pytest.mark.parametrize("n", [0, 1, 7, 8, 9, 17, 64, 1000])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_cpu_packing_equals_numpy_packbits(n, dtype):
    s = _spikes((n,), 100 + n, dtype)
    spike_b, s_dtype, s_shape, s_padding = float_spike_to_bool(s)
    assert spike_b.dtype == torch.uint8 and s_dtype == dtype and s_shape == s.shape and s_padding == 8 - n % 8
    assert np.array_equal(spike_b.numpy(), np.packbits(s.float().numpy().astype(np.uint8), bitorder="little"))
    back = bool_spike_to_float(spike_b, s_dtype, s_shape, s_padding)
    assert back.dtype == dtype and bits_equal(back, s)


def test_shape_is_restored_and_other_dtypes_are_refused():
    s = _spikes((3, 5, 7), 1)
    assert bits_equal(bool_spike_to_float(*float_spike_to_bool(s)), s)
    with pytest.raises(NotImplementedError):
        float_spike_to_bool(s.double())
    with pytest.raises(NotImplementedError):
        bool_spike_to_float(torch.zeros(2, dtype=torch.uint8), torch.int32, torch.Size([16]))


@pytest.mark.parametrize("level", [0, 1])
def test_cache_balances_repeated_stores(level, monkeypatch):
    monkeypatch.setattr(configure, "save_bool_spike_level", level)
    spike = (torch.arange(17) % 3 == 0).float()
    cache = BoolTensorCache()
    first, second = cache.store_bool(spike), cache.store_bool(spike)
    assert first == second == tensor_key(spike) and len(cache.cache) == 1
    payload = cache.cache[first][0]
    assert payload[1].dtype == (torch.bool if level == 0 else torch.uint8)
    assert payload[1].numel() == (17 if level == 0 else 3)
    assert torch.equal(cache.get_float(first, spike.shape), spike) and len(cache.cache) == 1
    # the form chosen at store time is the one read back, whatever the switch says by then
    monkeypatch.setattr(configure, "save_bool_spike_level", 1 - level)
    assert torch.equal(cache.get_float(second, spike.shape), spike) and len(cache.cache) == 0
    with pytest.raises(KeyError):
        cache.get_float(first, spike.shape)
    monkeypatch.setattr(configure, "save_bool_spike_level", 2)
    with pytest.raises(NotImplementedError):
        cache.store_bool(spike)


def test_tensor_key_names_the_elements_not_the_object():
    base = torch.zeros(4, 6)
    assert tensor_key(base) == tensor_key(base.view(24)) == (base.data_ptr(), base.data_ptr() + 23 * 4, 24)
    assert tensor_key(base[1:]) != tensor_key(base[:3])
    t = base.t()  # non-contiguous: last element of the view is the last element of the storage here
    assert tensor_key(t) == (base.data_ptr(), base.data_ptr() + 23 * 4, 24)
    assert tensor_key(torch.zeros(0)) [2] == 0


def test_cpu_tensors_and_string_paddings_run_the_plain_torch_functions(monkeypatch):
    def forbidden(*a, **k):
        raise AssertionError("the cache must not be used")

    monkeypatch.setattr(BOOL_TENSOR_CACHE, "store_bool", forbidden)
    s, w, b = _spikes((4, 6), 2).requires_grad_(), seeded_randn((5, 6), 3).requires_grad_(), seeded_randn((5,), 4)
    assert bits_equal(spike_op.spike_linear(s, w, b).detach(), F.linear(s, w, b).detach())
    img, k = _spikes((2, 3, 8, 8), 5), seeded_randn((4, 3, 3, 3), 6)
    assert bits_equal(spike_op.spike_conv2d(img, k, None, 1, "same"), F.conv2d(img, k, None, 1, "same"))
    layer = spike_op.SpikeConv1d(3, 4, 3, padding=1, padding_mode="circular")
    ref = nn.Conv1d(3, 4, 3, padding=1, padding_mode="circular")
    ref.load_state_dict(layer.state_dict())
    seq = _spikes((2, 3, 9), 7)
    assert bits_equal(layer(seq).detach(), ref(seq).detach())
    assert isinstance(spike_op.SpikeLinear(6, 5), nn.Linear) and isinstance(spike_op.SpikeConv3d(1, 1, 1), nn.Conv3d)


# ---- GPU ---------------------------------------------------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 8, 17, 4096, 100003])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_gpu_packing_equals_the_cpu_bytes(n, dtype):
    s = _spikes((n,), 200 + n, dtype)
    want = float_spike_to_bool(s)
    got = float_spike_to_bool(s.cuda())
    assert got[0].is_cuda and bits_equal(got[0].cpu(), want[0]) and got[1:] == want[1:]
    back = bool_spike_to_float(got[0], *got[1:])
    assert back.is_cuda and back.dtype == dtype and bits_equal(back.cpu(), s)


def _held_by_autograd(fn):
    held = []
    with torch.autograd.graph.saved_tensors_hooks(lambda t: held.append(t) or t, lambda t: t):
        out = fn()
    return out, held


@pytest.mark.gpu
@pytest.mark.parametrize("level", [0, 1])
@pytest.mark.parametrize("bias", [False, True])
def test_spike_linear_matches_linear_and_holds_no_float_spikes(level, bias, monkeypatch):
    monkeypatch.setattr(configure, "save_bool_spike_level", level)
    s = _spikes((8, 7, 32), 8).cuda()
    w, b = seeded_randn((16, 32), 9).cuda(), (seeded_randn((16,), 10).cuda() if bias else None)
    g = seeded_randn((8, 7, 16), 11).cuda()
    leaves = [t.clone().requires_grad_() for t in (s, w)] + ([b.clone().requires_grad_()] if bias else [None])
    refs = [t.clone().requires_grad_() for t in (s, w)] + ([b.clone().requires_grad_()] if bias else [None])
    out, held = _held_by_autograd(lambda: spike_op.spike_linear(*leaves))
    assert all(t.shape != s.shape for t in held)  # only the weight; the spikes sit in the cache as bool or bits
    entry = next(iter(BOOL_TENSOR_CACHE.cache.values()))[0]
    assert entry[1].numel() * entry[1].element_size() == (s.numel() if level == 0 else s.numel() // 8)
    want = F.linear(*refs)
    assert bits_equal(out.detach().cpu(), want.detach().cpu())
    out.backward(g)
    want.backward(g)
    assert len(BOOL_TENSOR_CACHE.cache) == 0
    for a, r in zip(leaves, refs):
        if a is not None:
            torch.testing.assert_close(a.grad, r.grad, rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("level", [0, 1])
@pytest.mark.parametrize("dim,shape,kshape,kw", [
    (1, (4, 3, 33), (5, 3, 3), dict(stride=2, padding=1)),
    (2, (4, 4, 14, 14), (6, 2, 3, 3), dict(padding=1, groups=2)),
    (2, (2, 3, 9, 9), (4, 3, 3, 3), dict(dilation=2, padding=(2, 0))),
    (3, (2, 2, 5, 6, 7), (3, 2, 3, 3, 3), dict(padding=1)),
])
def test_spike_convolutions_match_torch(level, dim, shape, kshape, kw, monkeypatch):
    monkeypatch.setattr(configure, "save_bool_spike_level", level)
    mine = {1: spike_op.spike_conv1d, 2: spike_op.spike_conv2d, 3: spike_op.spike_conv3d}[dim]
    ref = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[dim]
    s, k, b = _spikes(shape, 12).cuda(), seeded_randn(kshape, 13).cuda(), seeded_randn((kshape[0],), 14).cuda()
    a = [t.clone().requires_grad_() for t in (s, k, b)]
    r = [t.clone().requires_grad_() for t in (s, k, b)]
    out, held = _held_by_autograd(lambda: mine(*a, **kw))
    assert all(t.shape != s.shape for t in held)
    want = ref(*r, **kw)
    torch.testing.assert_close(out.detach(), want.detach(), rtol=1e-5, atol=1e-5)
    g = seeded_randn(tuple(out.shape), 15).cuda()
    out.backward(g)
    want.backward(g)
    assert len(BOOL_TENSOR_CACHE.cache) == 0
    for x, y in zip(a, r):
        torch.testing.assert_close(x.grad, y.grad, rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
def test_one_spike_tensor_feeding_two_layers_is_stored_once(monkeypatch):
    monkeypatch.setattr(configure, "save_bool_spike_level", 1)
    torch.manual_seed(16)
    left, right = spike_op.SpikeConv2d(3, 4, 3, padding=1).cuda(), spike_op.SpikeLinear(8, 5).cuda()
    s = _spikes((2, 3, 8, 8), 17).cuda().requires_grad_()
    out = left(s).sum() + right(s).sum()
    assert len(BOOL_TENSOR_CACHE.cache) == 1 and next(iter(BOOL_TENSOR_CACHE.cache.values()))[1] == 2
    out.backward()
    assert len(BOOL_TENSOR_CACHE.cache) == 0 and s.grad is not None
    # only a gradient for the bias: the spikes are not stored at all
    frozen = spike_op.SpikeConv2d(3, 4, 3).cuda()
    frozen.weight.requires_grad_(False)
    frozen(s.detach()).sum().backward()
    assert len(BOOL_TENSOR_CACHE.cache) == 0 and frozen.bias.grad is not None


@pytest.mark.gpu
def test_operators_pass_opcheck():
    s, w, b = _spikes((6, 32), 18).cuda().requires_grad_(), seeded_randn((16, 32), 19).cuda().requires_grad_(), None
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    torch.library.opcheck(spike_op.hip_spike_linear_forward, (s, w, b), test_utils=tests)
    img, k = _spikes((2, 3, 8, 8), 20).cuda().requires_grad_(), seeded_randn((4, 3, 3, 3), 21).cuda().requires_grad_()
    torch.library.opcheck(spike_op.hip_spike_convolution_forward, (img, k, None, [1, 1], [1, 1], [1, 1], 1), test_utils=tests)
    BOOL_TENSOR_CACHE.cache.clear()  # opcheck runs forwards whose backwards it never calls
