"""The contraction fused with the attention's LIF (``sjhip_ssa_lif_forward_packed`` / ``_backward_packed``) against the
separate kernels it stands for: ``sjhip_ssa_forward_packed`` followed by the neuron forward, and the neuron backward
followed by ``sjhip_ssa_backward_packed``.  Forward: spikes, ``h_seq`` and ``v_last`` bit for bit (the contraction is
exact and the neuron runs the same instructions).  Backward: the neuron's recurrence may fuse multiply-adds differently
in the two kernels, so 1e-6 relative to the largest gradient; the float64 oracle of the whole block is compared in
``tests/test_hip_conv_bn_lif.py``."""

import pytest
import torch

from spikingjelly_amd import configure
from spikingjelly_amd.activation_based import functional, layer

from helpers import bits_equal

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mods():
    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    from spikingjelly_amd.activation_based.hip_kernel import attention_kernel as A, compress, library as L, neuron_kernel as K

    L.load()
    return A, K, L, compress


def _bits(compress, T, B, H, C, Lp, seed, rate):
    g = torch.Generator().manual_seed(seed)
    qkv = (torch.rand((T * B, 3, H, C, Lp), generator=g) < rate).float().cuda()
    packed = compress.bit_spike_compress(qkv.flatten())
    bits = packed[0] if isinstance(packed, (tuple, list)) else packed
    return qkv, bits.view(torch.uint8).flatten()


def _rate(C, Lp):
    """Spike rate of q / k / v at which the contraction's output (0.125 * C * Lp * rate^3 on average) straddles the
    threshold, so that the neuron fires in some places and not in others."""
    return (5.0 / (C * Lp)) ** (1.0 / 3.0)


def _separate(A, K, L, qkv_bits, v_init, T, B, H, C, Lp, scale, tau, v_th, v_reset, flags, neuron_id=None):
    out = A._ssa_packed(qkv_bits, None, torch.float32, T * B, H, C, Lp, scale)
    x = out.view(T, B * H * C * Lp)
    spikes, _, v_last, h = K._run_forward(neuron_id if neuron_id is not None else L.NEURON_LIF, x, v_init, None, tau, v_th,
                                          v_reset, flags, False, True)
    return out, spikes, h, v_last


SHAPES = [(4, 3, 12, 32, 196), (1, 2, 2, 32, 64), (5, 2, 3, 48, 64), (3, 2, 2, 64, 100), (2, 1, 1, 8, 12), (2, 2, 1, 32, 256),
          (4, 2, 12, 64, 196)]


@pytest.mark.parametrize("T,B,H,C,Lp", SHAPES)
@pytest.mark.parametrize("soft,decay_input,tau", [(False, True, 2.0), (True, False, 3.0), (False, False, 2.0)])
def test_forward_equals_contraction_then_neuron(mods, T, B, H, C, Lp, soft, decay_input, tau):
    A, K, L, compress = mods
    _, bits = _bits(compress, T, B, H, C, Lp, 3 + Lp, _rate(C, Lp))
    flags = K._flags(soft, True, decay_input, 0)
    v_th, v_reset, scale = 0.5, 0.0, 0.125
    N = B * H * C * Lp
    for v_init in (torch.zeros(1, device="cuda").expand(N), torch.rand(N, device="cuda") * 0.4):
        out, spikes, h, v_last = _separate(A, K, L, bits, v_init, T, B, H, C, Lp, scale, tau, v_th, v_reset, flags)
        keep, broadcast = K._state_arg(v_init, True)
        params = K._params(tau, v_th, v_reset, 0.0, 0, flags | broadcast)
        got_s, got_h, got_v = A._ssa_lif_forward(bits, keep, params, T, B, H, C, Lp, scale, True)
        assert float(spikes.sum()) > 0 and float(spikes.mean()) < 1
        assert bits_equal(got_s.view(T, N), spikes)
        assert bits_equal(got_h.view(T, N), h)
        assert bits_equal(got_v.view(N), v_last)
        # inference: no h_seq
        got_s2, none_h, got_v2 = A._ssa_lif_forward(bits, keep, params, T, B, H, C, Lp, scale, False)
        assert none_h is None and bits_equal(got_s2, got_s) and bits_equal(got_v2, got_v)


def test_forward_if_neuron(mods):
    A, K, L, compress = mods
    T, B, H, C, Lp = 3, 2, 2, 32, 64
    _, bits = _bits(compress, T, B, H, C, Lp, 9, _rate(C, Lp) * 1.2)
    flags = K._flags(False, True, True, 0)
    N = B * H * C * Lp
    v_init = torch.zeros(1, device="cuda").expand(N)
    out, spikes, h, v_last = _separate(A, K, L, bits, v_init, T, B, H, C, Lp, 0.125, 2.0, 1.0, 0.0, flags, L.NEURON_IF)
    keep, broadcast = K._state_arg(v_init, True)
    params = K._params(2.0, 1.0, 0.0, 0.0, 0, flags | broadcast)
    spk = torch.empty((T, B, H, C, Lp), device="cuda")
    hh = torch.empty_like(spk)
    vl = torch.empty((B, H, C, Lp), device="cuda")
    import ctypes
    rc = L.load().sjhip_ssa_lif_forward_packed(L.NEURON_IF, ctypes.byref(params), T, B, H, C, Lp, 0.125, bits.data_ptr(),
                                               keep.data_ptr(), spk.data_ptr(), hh.data_ptr(), vl.data_ptr(),
                                               L.current_stream_ptr(spk.device))
    L.check(rc, "ssa_lif_forward_packed")
    assert bits_equal(spk.view(T, N), spikes) and bits_equal(hh.view(T, N), h) and bits_equal(vl.view(N), v_last)


@pytest.mark.parametrize("T,B,H,C,Lp", SHAPES)
@pytest.mark.parametrize("soft,detach,decay_input,tau,sg", [(False, True, True, 2.0, 1), (True, False, False, 3.0, 0),
                                                            (False, False, True, 2.0, 4)])
def test_backward_equals_neuron_then_contraction(mods, T, B, H, C, Lp, soft, detach, decay_input, tau, sg):
    A, K, L, compress = mods
    _, bits = _bits(compress, T, B, H, C, Lp, 5 + Lp, _rate(C, Lp))
    flags = K._flags(soft, detach, decay_input, 0)
    v_th, v_reset, scale, alpha = 0.5, 0.0, 0.125, 2.0
    N = B * H * C * Lp
    v_init = torch.rand(N, device="cuda") * 0.4
    out, spikes, h, v_last = _separate(A, K, L, bits, v_init, T, B, H, C, Lp, scale, tau, v_th, v_reset, flags)
    g = torch.Generator(device="cuda").manual_seed(17)
    grad_spikes = torch.randn((T, N), device="cuda", generator=g)
    grad_v_last = torch.randn((N,), device="cuda", generator=g) * 0.3
    for gs, gvl in ((grad_spikes, None), (grad_spikes, grad_v_last), (None, grad_v_last)):
        gx, gvi, _ = K._run_backward(L.NEURON_LIF, gs, None, gvl, h, None, None, None, tau, v_th, v_reset, flags, sg, alpha,
                                     True)
        want = A._ssa_packed(bits, gx.view(T * B, H, C, Lp), torch.float32, T * B, H, C, Lp, scale)
        params = K._params(tau, v_th, v_reset, alpha, sg, flags)
        got, got_gvi = A._ssa_lif_backward(bits, h.view(T, B, H, C, Lp), gs, gvl, params, T, B, H, C, Lp, scale, True)
        scale_q = float(want.abs().max())
        assert scale_q > 0
        assert float((got - want).abs().max()) <= 1e-6 * scale_q
        assert float((got_gvi.view(N) - gvi).abs().max()) <= 1e-6 * max(float(gvi.abs().max()), 1e-30)


def test_unsupported_arguments_are_refused(mods):
    A, K, L, compress = mods
    import ctypes
    lib = L.load()
    params = K._params(2.0, 0.5, 0.0, 2.0, 1, 0)
    dummy = torch.zeros(64, device="cuda")
    args = (dummy.data_ptr(),) * 5
    # tokens not a multiple of 4; a neuron with more state than IF / LIF
    rc = lib.sjhip_ssa_lif_forward_packed(L.NEURON_LIF, ctypes.byref(params), 1, 1, 1, 8, 6, 0.125, *args, None)
    assert rc == -2 and b"tokens" in lib.sjhip_last_error()
    rc = lib.sjhip_ssa_lif_forward_packed(L.NEURON_PLIF, ctypes.byref(params), 1, 1, 1, 8, 8, 0.125, *args, None)
    assert rc == -2 and b"IF and LIF" in lib.sjhip_last_error()
    rc = lib.sjhip_ssa_lif_backward_packed(L.NEURON_LIF, ctypes.byref(params), 1, 1, 1, 8, 8, 0.125, dummy.data_ptr(), None,
                                           None, None, dummy.data_ptr(), None, None)
    assert rc == -1 and b"NULL" in lib.sjhip_last_error()


@pytest.mark.parametrize("dim,heads,T,B,tokens", [(384, 12, 4, 2, 196), (96, 3, 3, 2, 64), (128, 2, 2, 2, 100)])
def test_block_with_the_fused_neuron_equals_the_block_without(monkeypatch, dim, heads, T, B, tokens):
    """``SpikingSelfAttention`` with ``configure.hip_fuse_ssa_lif`` on and off: the same spikes out, the same state in
    all three neurons, gradients within 1e-6 of the largest (two calls in a row, the second continuing the state)."""
    torch.manual_seed(5)
    block = layer.SpikingSelfAttention(dim, heads, backend="hip")
    with torch.no_grad():  # batch-norm offsets near the thresholds, so that all three neurons fire in places
        for bn in (block.qkv_conv_bn[1], block.proj_conv_bn[1]):
            bn.weight.normal_(1.0, 0.2)
            bn.bias.normal_(0.9, 0.3)
    block = block.cuda()
    x1 = torch.randn(T, B, dim, tokens, device="cuda") * 2.0
    x2 = torch.randn(T, B, dim, tokens, device="cuda") * 2.0
    g = torch.randn(T, B, dim, tokens, device="cuda")
    results = []
    for flag in (True, False):
        monkeypatch.setattr(configure, "hip_fuse_ssa_lif", flag)
        functional.reset_net(block)
        block.zero_grad(set_to_none=True)
        for bn in (block.qkv_conv_bn[1], block.proj_conv_bn[1]):
            bn.reset_running_stats()
        xa = x1.clone().requires_grad_()
        y1 = block(xa)
        y2 = block(x2)  # continues from the stored potentials
        (y1 * g).sum().backward()
        results.append((y1.detach(), y2.detach(), xa.grad.clone(), [p.grad.clone() for p in block.parameters()],
                        block.attn_lif.v.clone(), block.qkv_lif.v.clone()))
    a, b = results
    assert 0.02 < float(a[0].mean()) < 0.9 and float(a[4].detach().abs().sum()) > 0
    assert bits_equal(a[0], b[0]) and bits_equal(a[1], b[1])
    assert bits_equal(a[4].reshape(-1), b[4].reshape(-1)) and bits_equal(a[5].reshape(-1), b[5].reshape(-1))
    for ga, gb in [(a[2], b[2])] + list(zip(a[3], b[3])):
        assert float((ga - gb).abs().max()) <= 2e-6 * max(float(gb.abs().max()), 1e-30)
