"""The fused convolution / batch norm / LIF chain at the width of BASELINE configs[4] (D = 384, 12 heads, T = 4, 196
tokens) against the float64 oracle (``oracle/conv_bn_lif_oracle.py``) computed on the host.

At this size some membrane potentials always lie within rounding distance of a threshold (about two per hundred
thousand neurons at a margin of 1e-5), so the bar is: spikes equal wherever the oracle's ``|h - v_th|`` exceeds the
margin, few neurons inside it (counted, printed and bounded), gradients compared where no neuron inside the margin
feeds them, and the disagreement with float64 no larger than that of the same modules with torch's own convolution and
batch norm around the hip neurons (``configure.hip_fuse_conv_bn_lif = False``).
Reference semantics: fp32 ``Conv1d(k=1)`` -> ``BatchNorm1d`` -> ``LIFNode``, layer/attention.py:310-329, 370-384.
"""

import pytest
import torch

from oracle import conv_bn_lif_oracle as co
from oracle import neuron_oracle as no
from spikingjelly_amd import configure
from spikingjelly_amd.activation_based import functional, layer

from helpers import seeded_randn

pytestmark = pytest.mark.gpu

MARGIN = 1e-5
# The exact comparison of whole (step, sample) slabs of the block's output uses a narrower margin, or no slab of this
# size would be free of neurons inside it: 2e-6 is twice the error bound of the convolution at this depth (2^-23 of
# sum |w||x|, about 1e-6 for 384 Kaiming-uniform weights times unit-variance inputs; batch norm has unit scale here).
PIN_MARGIN = 2e-6
DIM, HEADS, T, TOKENS = 384, 12, 4, 196


def _inside(h, v_th, margin=MARGIN):
    """Neurons whose float64 membrane potential is within the margin of the threshold (exact ties excluded: they occur
    in the attention neuron, whose arithmetic on multiples of 1/8 is exact in fp32 and float64 alike)."""
    d = (h - v_th).abs()
    return (d <= margin) & (d != 0)


@pytest.fixture(scope="module")
def C():
    from spikingjelly_amd.activation_based.hip_kernel import conv_bn_lif, library

    library.load()
    return conv_bn_lif


@pytest.mark.parametrize("split", ["f16", "bf16"])
def test_qkv_chain_at_width_384_against_float64(C, split, monkeypatch):
    """``conv_bn_lif`` with the qkv convolution's shape (W [1152, 384], contraction depth 384): every spike outside the
    margin equals the oracle's, the gradients agree where no neuron inside the margin feeds them, and torch's fp32
    convolution + batch norm in front of the same neuron kernel is not closer to float64."""
    from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K

    monkeypatch.setattr(configure, "hip_conv_split", split)
    B, Cin, Cout = 8, DIM, 3 * DIM
    x = seeded_randn((T, B, Cin, TOKENS), 71, 0.0, 1.0)
    torch.manual_seed(72)
    w = torch.nn.Conv1d(Cin, Cout, 1, bias=False).weight.detach()[:, :, 0].clone()  # Kaiming-uniform, as the module has it
    gamma, beta = seeded_randn((Cout,), 73, 1.0, 0.2), seeded_randn((Cout,), 74, 0.9, 0.3)
    gs = seeded_randn((T, B, Cout, TOKENS), 75)
    x64, w64 = x.double().requires_grad_(), w.double().requires_grad_()
    g64, b64 = gamma.double().requires_grad_(), beta.double().requires_grad_()
    ref = co.conv_bn_lif(x64, w64, g64, b64, torch.zeros(Cout, dtype=torch.float64), torch.ones(Cout, dtype=torch.float64),
                         True, torch.zeros((B, Cout, TOKENS), dtype=torch.float64), detach_reset=True)
    ref["spike_seq"].backward(gs.double())
    inside = _inside(ref["h_seq"].detach(), 1.0)
    n_inside = int(inside.sum())
    print(f"\nqkv chain {split}: {n_inside} of {inside.numel()} neuron-steps within {MARGIN} of the threshold")
    assert n_inside < 1e-4 * inside.numel()

    spec = (2.0, 1.0, 0.0, K._flags(False, True, True, 0), no.SG_IDS["sigmoid"], 4.0)

    def run(fused):
        xd, wd = x.cuda().requires_grad_(), w.cuda().requires_grad_()
        gd, bd = gamma.cuda().requires_grad_(), beta.cuda().requires_grad_()
        rm, rv = torch.zeros(Cout, device="cuda"), torch.ones(Cout, device="cuda")
        v0 = torch.zeros((1,), device="cuda").expand(B, Cout, TOKENS)
        if fused:
            spikes, _ = C.conv_bn_lif(xd, wd, gd, bd, v0, (rm, rv, True, 0.1, 1e-5), spec, False)
        else:  # torch's operators around the same neuron kernel
            y = torch.nn.functional.conv1d(xd.flatten(0, 1), wd[:, :, None])
            z = torch.nn.functional.batch_norm(y, rm, rv, gd, bd, True, 0.1, 1e-5).view(T, B, Cout, TOKENS)
            spikes = functional.lif_multi_step_hip(z, torch.zeros((B, Cout, TOKENS), device="cuda"), 2.0, True, 1.0, 0.0,
                                                   _sigmoid(), True)[0]
        spikes.backward(gs.cuda())
        return spikes.detach().cpu().double(), xd.grad.cpu().double(), wd.grad.cpu().double(), gd.grad.cpu().double(), \
            bd.grad.cpu().double(), rm.cpu().double(), rv.cpu().double()

    results = {}
    for fused in (True, False):
        s, dx, dw, dg, db, rm, rv = run(fused)
        wrong = s != ref["spike_seq"].detach()
        assert not bool((wrong & ~inside).any()), "a spike outside the margin differs from float64"
        # a neuron inside the margin may fire differently; its gradient then differs at its own column (sample, token)
        flipped_cols = wrong.any(dim=2).any(dim=0)          # [B, L]
        clean = ~flipped_cols[None, :, None, :].expand_as(dx)
        scale = float(x64.grad.abs().max())
        err_dx = float(((dx - x64.grad).abs() * clean).max()) / scale
        err_dw = float((dw - w64.grad).abs().max() / w64.grad.abs().max())
        err_dg = float((dg - g64.grad).abs().max() / g64.grad.abs().max())
        err_db = float((db - b64.grad).abs().max() / b64.grad.abs().max())
        err_rm = float((rm - ref["running_mean"].detach()).abs().max())
        err_rv = float((rv - ref["running_var"].detach()).abs().max())
        results[fused] = (int(wrong.sum()), err_dx, err_dw, err_dg, err_db, err_rm, err_rv)
        print(f"  {'fused' if fused else 'torch conv + bn'}: {int(wrong.sum())} spikes differ (all inside the margin); "
              f"relative errors dx {err_dx:.2e} dW {err_dw:.2e} dgamma {err_dg:.2e} dbeta {err_db:.2e}; running mean {err_rm:.2e} var {err_rv:.2e}")
    wrong_f, dx_f, dw_f, dg_f, db_f, rm_f, rv_f = results[True]
    wrong_t, dx_t, dw_t, dg_t, db_t, rm_t, rv_t = results[False]
    assert wrong_f <= n_inside
    assert dx_f < 2e-5 and rm_f < 1e-6 and rv_f < 1e-6
    # a flipped spike moves the weight and batch-norm gradients by that one neuron's share: 1e-4 of the largest entry
    assert dw_f < 2e-4 and dg_f < 2e-4 and db_f < 2e-4
    # no further from float64 than torch's own fp32 operators (twice their error, or the floor of a single flipped spike)
    assert dx_f <= 2 * dx_t + 2e-6 and dw_f <= 2 * dw_t + 1e-4 and dg_f <= 2 * dg_t + 1e-4 and db_f <= 2 * db_t + 1e-4


def _sigmoid():
    from spikingjelly_amd.activation_based import surrogate

    return surrogate.Sigmoid(4.0)


def _block(seed):
    torch.manual_seed(seed)
    block = layer.SpikingSelfAttention(DIM, HEADS, backend="hip")
    with torch.no_grad():
        for bn in (block.qkv_conv_bn[1], block.proj_conv_bn[1]):
            bn.weight.normal_(1.0, 0.2)
            bn.bias.normal_(0.9, 0.3)
    return block


def _params(block):
    p = {}
    for name, seq in (("qkv", block.qkv_conv_bn), ("proj", block.proj_conv_bn)):
        p[f"{name}_weight"] = seq[0].weight.detach()[:, :, 0].double().cpu().clone()
        p[f"{name}_gamma"] = seq[1].weight.detach().double().cpu().clone()
        p[f"{name}_beta"] = seq[1].bias.detach().double().cpu().clone()
        p[f"{name}_running_mean"] = seq[1].running_mean.double().cpu().clone()
        p[f"{name}_running_var"] = seq[1].running_var.double().cpu().clone()
    return p


@pytest.mark.parametrize("B", [8, 64])
def test_attention_block_at_width_384_against_float64(B, monkeypatch):
    """The whole block (training mode) at D = 384 with 12 heads.  A spike that differs in one layer changes what the
    layers behind it see for its whole sample, so the exact comparison is made per (step, sample) slab: a slab of the
    output none of whose neurons in any of the three layers, at this or an earlier step of the sample, lies inside the
    (narrower) pinning margin must equal the oracle's.  Over all slabs the fused path's share of differing output spikes must not exceed
    that of the unfused path (torch's convolution and batch norm around the hip neurons)."""
    block = _block(81).cuda().train()
    params = _params(block)
    x = seeded_randn((T, B, DIM, TOKENS), 82, 0.0, 1.0)
    with torch.no_grad():
        ref = co.attention_block(x.double(), params, HEADS, True)
    inside = torch.zeros((T, B), dtype=torch.bool)
    total_inside = 0
    for key, v_th in (("qkv_h", 1.0), ("attn_h", 0.5), ("proj_h", 1.0)):
        total_inside += int(_inside(ref[key], v_th).sum())
        inside |= _inside(ref[key], v_th, PIN_MARGIN).flatten(2).any(dim=2)
    dirty = inside.cummax(dim=0).values  # a sample stays unpinned from the first step with a neuron inside the margin
    clean = ~dirty
    n_neurons = sum(ref[k].numel() for k in ("qkv_h", "attn_h", "proj_h"))
    print(f"\nblock B={B}: {total_inside} of {n_neurons} neuron-steps within {MARGIN} of a threshold; "
          f"{int(clean.sum())} of {T * B} (step, sample) slabs hold no neuron within {PIN_MARGIN} and are compared exactly")
    assert total_inside < 1e-4 * n_neurons
    assert int(clean.sum()) >= 1

    rates = {}
    xd = x.cuda()
    for fused in (True, False):
        monkeypatch.setattr(configure, "hip_fuse_conv_bn_lif", fused)
        for bn, name in ((block.qkv_conv_bn[1], "qkv"), (block.proj_conv_bn[1], "proj")):
            bn.running_mean.copy_(params[f"{name}_running_mean"])
            bn.running_var.copy_(params[f"{name}_running_var"])
        functional.reset_net(block)
        with torch.no_grad():
            out = block(xd).cpu().double()
        wrong = out != ref["out"]
        if fused:  # (torch's fp32 convolution is not held to the pinning margin: its error at this depth can exceed it)
            assert not bool(wrong[clean].any()), "a slab without a neuron inside the pinning margin differs from float64"
        rates[fused] = float(wrong.double().mean())
        print(f"  {'fused' if fused else 'torch conv + bn'}: {int(wrong.sum())} of {wrong.numel()} output spikes differ ({rates[fused]:.2e})")
        if fused:
            for bn, name in ((block.qkv_conv_bn[1], "qkv"), (block.proj_conv_bn[1], "proj")):
                torch.testing.assert_close(bn.running_mean.cpu().double(), ref[f"{name}_running"][0], rtol=1e-4, atol=1e-5)
                torch.testing.assert_close(bn.running_var.cpu().double(), ref[f"{name}_running"][1], rtol=1e-4, atol=1e-5)
    assert 0.01 < float(ref["out"].mean()) < 0.9
    assert rates[True] < 5e-4
    assert rates[True] <= 2.0 * rates[False] + 2e-5
