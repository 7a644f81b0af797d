"""Full-size checks (BASELINE configs 2 to 5 at their real shapes) through size-independent properties.

Neurons are independent, so any subset of columns of the full-size GPU result must equal the C oracle
run on those columns alone -- that covers every address range of the 2.1 GB tensors without a 30 GB
CPU run.  Plus the invariants that hold element-wise: s == [h >= v_th], v == h where no spike,
v == v_reset where one, and a mean firing rate in the expected range.
"""

import numpy as np
import pytest
import torch

from helpers import require_device_memory, seeded_randn

pytestmark = pytest.mark.gpu

T, N = 16, 256 * 128 * 32 * 32


@pytest.mark.parametrize("t_steps,n_neurons", [(T, N), (T, N + 1024), (128, N // 8)],
                         ids=["config2", "row_stride_off_a_power_of_two", "T128_replayed_in_pieces"])
def test_config2_full_size_forward_backward(c_oracle, t_steps, n_neurons):
    """BASELINE config 2, the same element count with rows 4 KiB longer (a row stride that is not a power of two),
    and the same element count as 128 steps (the forward leaves checkpoints, the backward replays in pieces)."""
    from spikingjelly_amd.activation_based import neuron, surrogate

    require_device_memory(40)
    T, N = t_steps, n_neurons
    g = torch.Generator(device="cuda").manual_seed(1002)
    x = (torch.randn((T, N), generator=g, device="cuda") * 0.8 + 0.3).requires_grad_()
    gs = torch.randn((T, N), generator=g, device="cuda")
    gv = torch.randn((T, N), generator=g, device="cuda") * 0.1
    node = neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(2.0), step_mode="m", backend="hip",
                          store_v_seq=True)
    s = node(x)
    torch.autograd.backward([s, node.v_seq], [gs, gv])
    torch.cuda.synchronize()
    rate = float(s.detach().mean())
    assert 0.02 < rate < 0.08, rate

    # column subset: blocks at the start, the end and random places in between
    rng = np.random.default_rng(0)
    starts = np.concatenate([[0, N - 4096], rng.integers(0, N - 4096, size=30)])
    cols = torch.from_numpy(np.concatenate([np.arange(a, a + 4096) for a in starts])).cuda()
    xs = x.detach()[:, cols].cpu().numpy()
    es, ev, eh = c_oracle.forward_f32("lif", xs, np.zeros(xs.shape[1], np.float32), 2.0, True, 1.0, 0.0)
    assert np.array_equal(s.detach()[:, cols].cpu().numpy(), es)
    assert np.array_equal(node.v_seq.detach()[:, cols].cpu().numpy().view(np.int32), ev.view(np.int32))
    assert np.array_equal(node.v.detach()[cols].cpu().numpy().view(np.int32), ev[-1].view(np.int32))
    gx, _, _ = c_oracle.backward_f64("lif", gs[:, cols].cpu().numpy(), gv[:, cols].cpu().numpy(), None, eh, 0.5, True,
                                     1.0, 0.0, False, 1, 2.0)
    np.testing.assert_allclose(x.grad[:, cols].cpu().numpy(), gx, rtol=1e-5, atol=1e-6)

    # element-wise invariants over the whole tensors (v_seq doubles as h where no spike)
    v_seq = node.v_seq.detach()
    fired = s.detach() > 0
    assert bool((v_seq[fired] == 0.0).all())
    assert bool((v_seq[~fired] < 1.0).all())
    assert bool(torch.isfinite(x.grad).all())


def _column_blocks(n_cols: int, width: int = 4096, count: int = 30, seed: int = 0):
    rng = np.random.default_rng(seed)
    starts = np.concatenate([[0, n_cols - width], rng.integers(0, n_cols - width, size=count)])
    return np.concatenate([np.arange(a, a + width) for a in starts])


def test_config3_full_size_plif_bf16_fp32_state(c_oracle):
    """BASELINE config 3 at full size: ParametricLIF (init_tau=2, so k = 1/2 exactly), soft reset, Sigmoid(4),
    x [8,128,256,16,16] bf16 with fp32 state.  The C oracle runs the whole tensor (fp32 arithmetic on the
    bf16-representable inputs is the fp32-state semantics): every spike must match, stored v_seq must be the
    oracle's v rounded to bf16, grad_x agrees to bf16 accuracy, and the global dL/dw -- one scalar reduced
    over 67 M terms -- agrees with the float64 recurrence and is additive over a split of the neurons."""
    from spikingjelly_amd import configure
    from spikingjelly_amd.activation_based import functional, neuron, surrogate

    Tc, Nc = 8, 128 * 256 * 16 * 16
    g = torch.Generator().manual_seed(1003)
    x = (torch.randn((Tc, Nc), generator=g) * 1.0 + 0.2).bfloat16()
    gs = torch.randn((Tc, Nc), generator=torch.Generator().manual_seed(1103)).bfloat16()
    gv = (torch.randn((Tc, Nc), generator=torch.Generator().manual_seed(1203)) * 0.1).bfloat16()
    old = configure.hip_half_precision_mode
    configure.hip_half_precision_mode = "fp32_state"
    try:
        node = neuron.ParametricLIFNode(init_tau=2.0, v_reset=None, surrogate_function=surrogate.Sigmoid(4.0),
                                        step_mode="m", backend="hip", store_v_seq=True).cuda()
        xd = x.cuda().requires_grad_()
        s = node(xd)
        torch.autograd.backward([s, node.v_seq], [gs.cuda(), gv.cuda()])
        torch.cuda.synchronize()
        rate = float(s.detach().float().mean())
        assert 0.03 < rate < 0.09, rate

        es, ev, eh = c_oracle.forward_f32("plif", x.float().numpy(), np.zeros(Nc, np.float32), 0.5, True, 1.0, None)
        assert np.array_equal(s.detach().float().cpu().numpy(), es)
        assert torch.equal(node.v_seq.detach().cpu(), torch.from_numpy(ev).bfloat16())
        assert torch.equal(node.v.detach().cpu(), torch.from_numpy(ev[-1]).bfloat16())

        gx, _, gk = c_oracle.backward_f64("plif", gs.float().numpy(), gv.float().numpy(), None, eh, 0.5, True, 1.0, None,
                                          False, 0, 4.0, x_seq=x.float().numpy(), v_init=np.zeros(Nc, np.float32), v_seq=ev)
        cols = _column_blocks(Nc)
        np.testing.assert_allclose(xd.grad.float().cpu().numpy()[:, cols], gx[:, cols], rtol=1e-2, atol=2e-3)
        dw = float(node.w.grad)
        assert abs(dw - gk * 0.25) <= 2e-3 * abs(gk * 0.25) + 1e-3, (dw, gk * 0.25)  # dL/dw = dL/dk k (1 - k)

        # additivity of the reduction over a split of the neurons
        parts = []
        for lo, hi in ((0, Nc // 2), (Nc // 2, Nc)):
            functional.reset_net(node)
            node.w.grad = None
            xi = x[:, lo:hi].contiguous().cuda().requires_grad_()
            si = node(xi)
            torch.autograd.backward([si, node.v_seq], [gs[:, lo:hi].contiguous().cuda(), gv[:, lo:hi].contiguous().cuda()])
            parts.append(float(node.w.grad))
        assert abs(sum(parts) - dw) <= 1e-4 * abs(dw) + 1e-4, (parts, dw)
    finally:
        configure.hip_half_precision_mode = old


def test_config4_full_size_if_fp16_inference_and_packing():
    """BASELINE config 4 at full size: IF, soft reset, fp16, x [32,64,512,14,14] uniform[0,0.25); spikes are
    bit-packed and unpacked again.  Column blocks must equal the torch-ops oracle on the same half tensors;
    over the whole tensor the packed bytes must equal numpy.packbits of the spikes, the unpacked tensor the
    spikes, the fused packed-output kernel the two-kernel result, and the firing rate the input mean."""
    from oracle import neuron_oracle as no
    from spikingjelly_amd import configure
    from spikingjelly_amd.activation_based import functional
    from spikingjelly_amd.activation_based.hip_kernel.compress import bit_spike_compress, bit_spike_decompress

    Tc, Nc = 32, 64 * 512 * 14 * 14
    x = (torch.rand((Tc, Nc), generator=torch.Generator().manual_seed(1004)) * 0.25).half()
    old = configure.hip_half_precision_mode
    configure.hip_half_precision_mode = "torch"
    try:
        xd = x.cuda()
        v0 = torch.zeros(Nc, dtype=torch.float16, device="cuda")
        with torch.no_grad():
            s, v_next, _ = functional.if_multi_step_hip(xd, v0, 1.0, None, None)
            packed = bit_spike_compress(s)
            back = bit_spike_decompress(packed, s.shape, dtype=torch.float16)
            fused, v_next_f, _ = functional.if_multi_step_hip_packed(xd, v0, 1.0, None)
        torch.cuda.synchronize()
    finally:
        configure.hip_half_precision_mode = old
    assert packed.numel() == Tc * Nc // 8
    assert torch.equal(back, s)
    assert torch.equal(fused, packed) and torch.equal(v_next_f, v_next)
    s_cpu = s.cpu()
    assert np.array_equal(packed.cpu().numpy(), np.packbits(s_cpu.numpy().reshape(-1).astype(bool), bitorder="little"))
    rate = float(s_cpu.float().mean())
    assert 0.10 < rate < 0.125, rate  # tends to the input mean 0.125 once the membranes have charged

    cols = torch.from_numpy(_column_blocks(Nc, width=2048, count=14, seed=4))
    es, ev, _ = no.multi_step("if", x[:, cols], torch.zeros(cols.numel(), dtype=torch.float16), None, True, 1.0, None)
    assert torch.equal(s_cpu[:, cols], es)
    assert torch.equal(v_next.cpu()[cols], ev[-1])


def _config5_blocks():
    from spikingjelly_amd.activation_based import layer

    torch.manual_seed(1005)
    a = layer.SpikingSelfAttention(384, 12, backend="torch").cuda()
    b = layer.SpikingSelfAttention(384, 12, backend="hip").cuda()
    b.load_state_dict(a.state_dict())
    x = torch.randn((4, 64, 384, 196), generator=torch.Generator().manual_seed(1105)).cuda()
    g = torch.randn((4, 64, 384, 196), generator=torch.Generator().manual_seed(1205)).cuda()
    return a, b, x, g


def test_config5_full_size_block_matches_torch_backend(monkeypatch):
    """BASELINE config 5 at full size (T=4, B=64, 196 tokens, D=384, 12 heads): the block with backend='hip' and the
    convolution / batch-norm fusion switched off, against the same block with backend='torch' on the same device and
    weights.  Convolutions and batch norms are then the same torch kernels, the LIF kernels are bit-exact and the
    contraction is exact, so the output spikes must be identical; gradients agree to fp32 accuracy."""
    from spikingjelly_amd import configure
    from spikingjelly_amd.activation_based import functional

    from helpers import bits_equal

    monkeypatch.setattr(configure, "hip_fuse_conv_bn_lif", False)
    a, b, x, g = _config5_blocks()
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    ya = a(xa)
    ya.backward(g)
    yb = b(xb)
    yb.backward(g)
    torch.cuda.synchronize()
    assert 0.0 < float(ya.detach().mean()) < 0.5
    assert bits_equal(yb, ya)
    torch.testing.assert_close(xb.grad, xa.grad, rtol=1e-3, atol=1e-4)
    torch.testing.assert_close(b.proj_conv_bn[0].weight.grad, a.proj_conv_bn[0].weight.grad, rtol=1e-3, atol=1e-3)
    functional.reset_net(a)
    functional.reset_net(b)


def test_config5_full_size_fused_block_against_torch_backend():
    """The same comparison with the fused convolution / batch norm / LIF kernels (the default).  Two fp32 convolutions
    of different libraries differ in the last bits, so among the 290 million membrane potentials of the block a few
    hundred land on the other side of a threshold; each such spike changes the attention of its (sample, head) and with
    it the gradient of that sample's neighbourhood.  Expected values are therefore compared statistically: the output
    spikes differ in fewer than one in ten thousand positions, the gradients agree within fp32 tolerance on more than
    97 % of the elements and point the same way."""
    from spikingjelly_amd.activation_based import functional

    a, b, x, g = _config5_blocks()
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    ya = a(xa)
    ya.backward(g)
    yb = b(xb)
    yb.backward(g)
    torch.cuda.synchronize()
    assert 0.0 < float(ya.detach().mean()) < 0.5
    assert float((yb != ya).float().mean()) < 1e-4

    def agree(got, want, rtol, atol):
        close = (got - want).abs() <= atol + rtol * want.abs()
        cos = torch.nn.functional.cosine_similarity(got.flatten().double(), want.flatten().double(), dim=0)
        return float(close.float().mean()), float(cos)

    frac, cos = agree(xb.grad, xa.grad, 1e-3, 1e-4)
    assert frac > 0.97 and cos > 0.999, (frac, cos)
    for name in ("qkv_conv_bn", "proj_conv_bn"):
        frac, cos = agree(getattr(b, name)[0].weight.grad, getattr(a, name)[0].weight.grad, 1e-2, 1e-2)
        assert frac > 0.97 and cos > 0.999, (name, frac, cos)
    functional.reset_net(a)
    functional.reset_net(b)


def test_more_than_two_to_the_32_elements(c_oracle):
    """T x N beyond 2^32 elements (the reference's kernels index with 32-bit integers and refuse more than 2^31 - 1
    elements, cuda_kernel/cuda_utils.py:25-30): every element offset is 64-bit here.  Column blocks from every part of
    the range, the last columns included, against the C oracle, for the forward and the replaying backward."""
    from spikingjelly_amd.activation_based import neuron, surrogate

    require_device_memory(100)
    T_big, N_big = 16, (1 << 28) + 4096 * 3  # 4 295 163 904 elements per tensor, 17.2 GB in fp32
    g = torch.Generator(device="cuda").manual_seed(77)
    x = torch.empty((T_big, N_big), device="cuda")
    for t in range(T_big):  # row by row: the generator's own kernels need not cope with the full size
        x[t] = torch.randn((N_big,), generator=g, device="cuda") * 0.8 + 0.3
    x.requires_grad_()
    node = neuron.LIFNode(tau=2.0, surrogate_function=surrogate.ATan(2.0), step_mode="m", backend="hip", store_v_seq=False)
    s = node(x)
    rng = np.random.default_rng(1)
    starts = np.concatenate([[0, N_big - 4096, (1 << 28) - 2048], rng.integers(0, N_big - 4096, size=12)])
    cols = torch.from_numpy(np.concatenate([np.arange(a, a + 4096) for a in starts])).cuda()
    gs_cols = seeded_randn((T_big, cols.numel()), 78)
    gs = torch.zeros((T_big, N_big), device="cuda")
    gs[:, cols] = gs_cols.cuda()
    s.backward(gs)
    torch.cuda.synchronize()
    xs = x.detach()[:, cols].cpu().numpy()
    es, ev, eh = c_oracle.forward_f32("lif", xs, np.zeros(xs.shape[1], np.float32), 2.0, True, 1.0, 0.0)
    assert np.array_equal(s.detach()[:, cols].cpu().numpy(), es) and 0.02 < float(es.mean()) < 0.08
    assert np.array_equal(node.v.detach()[cols].cpu().numpy().view(np.int32), ev[-1].view(np.int32))
    # duplicate columns in `cols` (blocks may overlap) received the last write of gs_cols: read back what the kernel saw
    gx, _, _ = c_oracle.backward_f64("lif", gs[:, cols].cpu().numpy(), None, None, eh, 0.5, True, 1.0, 0.0, False, 1, 2.0)
    np.testing.assert_allclose(x.grad[:, cols].cpu().numpy(), gx, rtol=1e-5, atol=1e-6)
    # columns that received no upstream gradient have none
    probe = (1 << 27) + 12345
    assert probe not in set(cols.tolist()) and float(x.grad[:, probe].abs().max()) == 0.0
