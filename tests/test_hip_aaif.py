"""Activation-aware IF on the hip backend against the oracle and the torch backend (inference only).

Bars: spikes and membrane potentials bit-exact in fp32 and in every-op-rounded 16-bit mode, for scalar and
per-channel parameters at every position of the channel axis.
"""

import pytest
import torch

from oracle import neuron_oracle as no
from spikingjelly_amd import configure
from spikingjelly_amd.activation_based import functional, neuron

from helpers import bits_equal, require_device_memory, seeded_randn

pytestmark = pytest.mark.gpu


def _node(threshold, offset, channel_dim, v_reset, store_v_seq, backend):
    node = neuron.ActivationAwareIFNode(v_threshold=threshold, v_offset=offset, channel_dim=channel_dim, v_reset=v_reset,
                                        step_mode="m", backend=backend, store_v_seq=store_v_seq)
    return node.eval()


CASES = [  # step shape, channel_dim, threshold, offset
    ((4, 6, 5), -1, torch.tensor([1.0, 1.5, 2.0, 0.5, 0.75]), torch.tensor([0.0, 0.25, -0.25, 0.1, 0.0])),
    ((2, 3, 8, 8), 1, torch.tensor([1.0, 2.0, 0.6]), torch.tensor([0.0, 0.5, -0.1])),
    ((2, 3, 7, 9), 1, torch.tensor([1.0, 2.0, 0.6]), 0.25),            # odd inner size: channels change inside a vector
    ((8, 16), 0, 1.25, torch.linspace(-0.2, 0.2, 8)),                  # channel axis first, scalar threshold
    ((4, 64), -1, 1.5, 0.25),                                           # both scalar
    ((3, 37), -1, torch.linspace(0.5, 2.0, 37), 0.0),                   # ragged: element-wise kernel
]


@pytest.mark.parametrize("shape,channel_dim,threshold,offset", CASES)
@pytest.mark.parametrize("v_reset", [None, 0.25])
@pytest.mark.parametrize("store_v_seq", [False, True])
def test_fp32_bit_exact(shape, channel_dim, threshold, offset, v_reset, store_v_seq):
    T = 9
    x = seeded_randn((T,) + shape, 31 + len(shape), 0.35, 0.6)
    v0 = torch.full(shape, 0.0 if v_reset is None else v_reset)
    es, ev = no.activation_aware_if_multi_step(x, v0, threshold, offset, channel_dim, v_reset)
    assert 0.02 < float(es.mean()) < 0.9
    node = _node(threshold, offset, channel_dim, v_reset, store_v_seq, "hip").cuda()
    with torch.no_grad():
        s = node(x.cuda())
    assert bits_equal(s.cpu(), es) and bits_equal(node.v.cpu(), ev[-1])
    if store_v_seq:
        assert bits_equal(node.v_seq.cpu(), ev)
    # a second call continues from the carried state
    x2 = seeded_randn((T,) + shape, 77, 0.35, 0.6)
    es2, ev2 = no.activation_aware_if_multi_step(x2, ev[-1], threshold, offset, channel_dim, v_reset)
    with torch.no_grad():
        s2 = node(x2.cuda())
    assert bits_equal(s2.cpu(), es2) and bits_equal(node.v.cpu(), ev2[-1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("v_reset", [None, 0.25])
def test_16bit_modes(dtype, v_reset):
    shape, T = (2, 3, 8, 8), 12
    threshold, offset = torch.tensor([1.0, 2.1, 0.6]), torch.tensor([0.0, 0.3, -0.1])
    x = seeded_randn((T,) + shape, 5, 0.35, 0.6).to(dtype)
    v0 = torch.full(shape, 0.0 if v_reset is None else v_reset, dtype=dtype)
    old = configure.hip_half_precision_mode
    try:
        configure.hip_half_precision_mode = "torch"
        es, ev = no.activation_aware_if_multi_step(x, v0, threshold, offset, 1, v_reset)
        node = _node(threshold, offset, 1, v_reset, True, "hip").cuda()
        with torch.no_grad():
            s = node(x.cuda())
        assert bits_equal(s.cpu(), es) and bits_equal(node.v_seq.cpu(), ev)
        # fp32 state: parameters rounded to the storage dtype, arithmetic and carried v in fp32, stores rounded
        configure.hip_half_precision_mode = "fp32_state"
        es32, ev32 = no.activation_aware_if_multi_step(x.float(), v0.float(), threshold.to(dtype).float(),
                                                       offset.to(dtype).float(), 1, v_reset)
        node = _node(threshold, offset, 1, v_reset, True, "hip").cuda()
        with torch.no_grad():
            s = node(x.cuda())
        assert bits_equal(s.cpu(), es32.to(dtype)) and bits_equal(node.v_seq.cpu(), ev32.to(dtype))
    finally:
        configure.hip_half_precision_mode = old


def test_hip_backend_refuses_what_the_reference_kernel_backend_refuses():
    th = torch.tensor([1.0, 2.0])
    with pytest.raises(ValueError, match="step_mode='m'"):
        neuron.ActivationAwareIFNode(v_threshold=th, backend="hip")
    node = neuron.ActivationAwareIFNode(v_threshold=th, step_mode="m", backend="hip").cuda()
    x = torch.rand(3, 4, 2, device="cuda")
    with pytest.raises(RuntimeError, match="inference only"):
        node(x)
    node.eval()
    with pytest.raises(RuntimeError, match="autograd"):
        node(x.clone().requires_grad_())
    with pytest.raises(RuntimeError, match="ROCm device"):
        node(x.cpu())
    with pytest.raises(ValueError, match="channels"):
        node(torch.rand(3, 4, 5, device="cuda"))
    with torch.no_grad():
        assert node(x).shape == x.shape
    functional.reset_net(node)
    assert node.v == 0.0 and node.v_seq is None


def test_full_size_inference():
    """[T=16, B=64, C=128, 32, 32] fp32 with per-channel parameters: column blocks against the oracle."""
    require_device_memory(8)
    T, B, C, HW = 16, 64, 128, 1024
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn((T, B, C, HW), generator=g, device="cuda") * 0.5 + 0.2
    th = torch.linspace(0.5, 2.0, C)
    off = torch.linspace(-0.2, 0.2, C)
    node = neuron.ActivationAwareIFNode(v_threshold=th, v_offset=off, channel_dim=1, step_mode="m", backend="hip").cuda().eval()
    with torch.no_grad():
        s = node(x)
    assert 0.05 < float(s.mean()) < 0.6
    for b, c in ((0, 0), (17, 63), (63, 127)):
        es, ev = no.activation_aware_if_multi_step(x[:, b, c].cpu(), torch.zeros(HW), float(th[c]), float(off[c]), -1, None)
        assert bits_equal(s[:, b, c].cpu(), es) and bits_equal(node.v[b, c].cpu(), ev[-1])
