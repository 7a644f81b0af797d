"""Spiking self-attention on the matrix cores against the oracle (config 5 shape and edge shapes)."""

import pytest
import torch

from oracle import ssa_oracle
from spikingjelly_amd.activation_based import functional, layer
from spikingjelly_amd.activation_based.hip_kernel.attention_kernel import hip_ssa_backward, hip_ssa_forward

from helpers import bits_equal

pytestmark = pytest.mark.gpu


def _spikes(shape, seed, rate=0.2):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(shape, generator=g) < rate).float()


@pytest.mark.parametrize("S,H,C,L", [(6, 12, 32, 196), (3, 2, 32, 64), (2, 3, 48, 64), (2, 2, 64, 100), (1, 1, 8, 5),
                                     (2, 1, 32, 256), (1, 2, 33, 31), (3, 12, 64, 196)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_forward_is_exact(S, H, C, L, dtype):
    qkv = _spikes((S, 3, H, C, L), 7 + L, 0.5 if L * C < 2000 else 0.15)
    exact = ssa_oracle.ssa_exact(qkv, 0.125)
    out = hip_ssa_forward(qkv.to(dtype).cuda(), 0.125).cpu()
    assert out.dtype == dtype and out.shape == (S, H, C, L)
    if dtype == torch.float32:
        assert torch.equal(out.double(), exact)  # integer sums * 2^-3: exact in fp32
    else:
        assert bits_equal(out, exact.to(dtype))  # one rounding of the exact value
        if dtype == torch.bfloat16:
            assert bits_equal(out, ssa_oracle.ssa(qkv.to(dtype), 0.125))  # == torch's own bf16 matmul chain


def test_forward_maximal_sums_all_ones():
    qkv = torch.ones(1, 3, 1, 64, 100)
    out = hip_ssa_forward(qkv.cuda(), 0.125).cpu()
    assert torch.equal(out, torch.full((1, 1, 64, 100), 0.125 * 64 * 100))


@pytest.mark.parametrize("S,H,C,L", [(4, 12, 32, 196), (2, 3, 48, 64), (2, 2, 64, 100), (1, 2, 33, 31), (3, 12, 64, 196)])
def test_backward_matches_float64_autograd(S, H, C, L):
    qkv = _spikes((S, 3, H, C, L), 11 + L, 0.2)
    g = torch.Generator().manual_seed(5)
    grad_out = torch.randn((S, H, C, L), generator=g)
    ref_in = qkv.double().requires_grad_()
    ssa_oracle.ssa(ref_in, 0.125).backward(grad_out.double())
    got = hip_ssa_backward(qkv.cuda(), grad_out.cuda(), 0.125).cpu()
    torch.testing.assert_close(got.double(), ref_in.grad, rtol=1e-5, atol=1e-5)
    # through autograd of the forward op
    x = qkv.cuda().requires_grad_()
    hip_ssa_forward(x, 0.125).backward(grad_out.cuda())
    assert bits_equal(x.grad.cpu(), got)


def test_backward_bf16_storage():
    S, H, C, L = 2, 4, 32, 196
    qkv = _spikes((S, 3, H, C, L), 21, 0.2)
    grad_out = torch.randn((S, H, C, L), generator=torch.Generator().manual_seed(6)).bfloat16()
    ref_in = qkv.double().requires_grad_()
    ssa_oracle.ssa(ref_in, 0.125).backward(grad_out.double())
    got = hip_ssa_backward(qkv.bfloat16().cuda(), grad_out.cuda(), 0.125).cpu()
    torch.testing.assert_close(got.double(), ref_in.grad, rtol=1e-2, atol=1e-2)


def test_unsupported_shapes_raise():
    with pytest.raises(NotImplementedError, match="256 tokens"):
        hip_ssa_forward(torch.zeros(1, 3, 1, 32, 300, device="cuda"), 0.125)
    with pytest.raises(NotImplementedError):
        hip_ssa_forward(torch.zeros(1, 3, 1, 128, 16, device="cuda"), 0.125)
    with pytest.raises(RuntimeError, match="ROCm device"):
        hip_ssa_forward(torch.zeros(1, 3, 1, 32, 16), 0.125)


@pytest.mark.parametrize("fused", [False, True])
def test_block_hip_backend_equals_torch_backend_config5_reduced(fused, monkeypatch):
    """Config 5 at reduced batch: T=4, tokens 196, D=384, 12 heads, same weights, same device.  With torch's
    convolutions and batch norm around the hip neurons (``hip_fuse_conv_bn_lif = False``) the 1x1 convolutions are
    identical, the LIF kernels are bit-exact and the contraction is exact, so the hip block reproduces the torch block's
    spikes exactly and its gradients to fp32 accuracy.  With the library's own convolution GEMMs (the default) the
    pre-activations differ from torch's in the last bits, so a neuron within rounding of its threshold may fire
    differently; such a flip changes the gradients of its own sample (and, through the batch statistics, a few elements
    elsewhere): all but a few of the 8 samples must agree to fp32 accuracy in all but 1e-3 of their elements, and the
    output spikes in all but 1e-4 of the positions."""
    from spikingjelly_amd import configure

    monkeypatch.setattr(configure, "hip_fuse_conv_bn_lif", fused)
    torch.manual_seed(1005)
    a = layer.SpikingSelfAttention(384, 12, backend="torch").cuda()
    b = layer.SpikingSelfAttention(384, 12, backend="hip").cuda()
    b.load_state_dict(a.state_dict())
    x = torch.randn((4, 8, 384, 196), generator=torch.Generator().manual_seed(1105)).cuda()
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    ya, yb = a(xa), b(xb)
    assert 0.0 < float(ya.detach().mean()) < 0.5
    g = torch.randn(ya.shape, generator=torch.Generator().manual_seed(7)).cuda()
    ya.backward(g)
    yb.backward(g)
    wa, wb = a.qkv_conv_bn[0].weight.grad, b.qkv_conv_bn[0].weight.grad
    if not fused:
        assert bits_equal(yb, ya)
        torch.testing.assert_close(xb.grad, xa.grad, rtol=1e-3, atol=1e-4)
        torch.testing.assert_close(wb, wa, rtol=1e-3, atol=1e-3)
    else:
        assert float((yb != ya).float().mean()) < 1e-4
        close = torch.isclose(xb.grad, xa.grad, rtol=1e-3, atol=1e-4)
        off = (~close).float().transpose(0, 1).flatten(1).mean(1)    # fraction of elements off, per batch sample
        assert int((off > 1e-3).sum()) <= 2, off   # (the batch statistics carry a trace of a flip into the other samples)
        assert float((~close).float().mean()) < 0.05
        scale = float(wa.abs().max())
        assert float((wb - wa).abs().max()) < 0.05 * scale            # a flipped spike moves a weight gradient a little
    functional.reset_net(a)
    functional.reset_net(b)
