"""Pins of ``oracle/conv_bn_lif_oracle.py`` (CPU): its plain-algebra convolution and batch norm against torch's own
``nn.Conv1d`` / ``nn.BatchNorm1d`` modules (the operators the reference block is built from, layer/attention.py:310-329),
the running-statistics update included, and the whole block against this package's ``backend='torch'`` module."""

import pytest
import torch
import torch.nn as nn

from oracle import conv_bn_lif_oracle as co
from spikingjelly_amd.activation_based import layer

from helpers import seeded_randn


def test_pointwise_convolution_is_conv1d_with_kernel_size_one():
    x = seeded_randn((3, 2, 6, 8), 1, 0.0, 1.0, torch.float64)
    conv = nn.Conv1d(6, 10, 1, bias=False).double()
    want = conv(x.flatten(0, 1)).view(3, 2, 10, 8)
    torch.testing.assert_close(co.pointwise_conv(x, conv.weight.detach()[:, :, 0]), want.detach(), rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("training", [True, False])
def test_batch_norm_is_torch_batch_norm(training):
    y = seeded_randn((3, 2, 5, 8), 2, 0.3, 2.0, torch.float64)
    bn = nn.BatchNorm1d(5).double()
    with torch.no_grad():
        bn.weight.copy_(seeded_randn((5,), 3, 1.0, 0.2, torch.float64))
        bn.bias.copy_(seeded_randn((5,), 4, 0.0, 0.2, torch.float64))
        bn.running_mean.copy_(seeded_randn((5,), 5, 0.0, 0.2, torch.float64))
        bn.running_var.copy_(seeded_randn((5,), 6, 1.0, 0.1, torch.float64).abs())
    rm, rv = bn.running_mean.clone(), bn.running_var.clone()
    bn.train(training)
    want = bn(y.flatten(0, 1)).view(y.shape).detach()
    z, new_rm, new_rv = co.batch_norm(y, bn.weight.detach(), bn.bias.detach(), rm, rv, training, bn.momentum, bn.eps)
    torch.testing.assert_close(z, want, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(new_rm, bn.running_mean, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(new_rv, bn.running_var, rtol=1e-12, atol=1e-12)


def test_batch_norm_closed_form_on_two_values():
    # one channel holding -1 and 3: mean 1, biased variance 4, so z = -+1 / sqrt(1 + eps / 4) up to gamma, beta
    y = torch.tensor([-1.0, 3.0], dtype=torch.float64).view(1, 2, 1, 1)
    z, rm, rv = co.batch_norm(y, torch.tensor([2.0], dtype=torch.float64), torch.tensor([0.5], dtype=torch.float64),
                              torch.zeros(1, dtype=torch.float64), torch.ones(1, dtype=torch.float64), True, 0.1, 0.0)
    assert z.flatten().tolist() == [-1.5, 2.5]
    assert rm.item() == pytest.approx(0.1) and rv.item() == pytest.approx(0.9 + 0.1 * 8.0)  # unbiased variance 8


@pytest.mark.parametrize("training", [True, False])
def test_attention_block_is_the_torch_backend_module(training):
    torch.manual_seed(7)
    dim, heads, T, B, tokens = 16, 2, 3, 2, 8
    block = layer.SpikingSelfAttention(dim, heads, backend="torch").double()
    with torch.no_grad():
        for bn in (block.qkv_conv_bn[1], block.proj_conv_bn[1]):
            bn.running_mean.normal_(0.0, 0.1)
            bn.running_var.uniform_(0.5, 1.5)
            bn.weight.normal_(1.0, 0.2)
            bn.bias.normal_(0.9, 0.3)
    params = {}
    for name, seq in (("qkv", block.qkv_conv_bn), ("proj", block.proj_conv_bn)):
        params[f"{name}_weight"] = seq[0].weight.detach()[:, :, 0].clone()
        params[f"{name}_gamma"], params[f"{name}_beta"] = seq[1].weight.detach().clone(), seq[1].bias.detach().clone()
        params[f"{name}_running_mean"], params[f"{name}_running_var"] = seq[1].running_mean.clone(), seq[1].running_var.clone()
    block.train(training)
    x = seeded_randn((T, B, dim, tokens), 8, 0.0, 2.0, torch.float64)
    want = block(x).detach()
    got = co.attention_block(x, params, heads, training)
    assert torch.equal(got["out"], want)
    assert 0.02 < float(want.mean()) < 0.9
    torch.testing.assert_close(got["qkv_running"][0], block.qkv_conv_bn[1].running_mean, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(got["proj_running"][1], block.proj_conv_bn[1].running_var, rtol=1e-12, atol=1e-12)
