"""Spike bit-packing on the GPU against the oracle: bytes bit-exact, round trip exact."""

import numpy as np
import pytest
import torch

from oracle import bitpack_oracle
from spikingjelly_amd.activation_based import neuron, surrogate
from spikingjelly_amd.activation_based.hip_kernel.compress import bit_spike_compress, bit_spike_decompress
from spikingjelly_amd.activation_based.memopt import BitSpikeCompressor

from helpers import seeded_rand

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 7, 8, 9, 15, 16, 17, 31, 33, 63, 64, 65, 255, 256, 1000, 4096, 4097, 65536 + 5, (1 << 20) + 3]
DTYPES = [torch.float32, torch.float16, torch.bfloat16, torch.uint8, torch.bool]


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("n", SIZES)
def test_pack_matches_oracle_and_round_trips(dtype, n):
    rng = np.random.default_rng(n)
    bits = rng.random(n) < 0.2
    src = torch.from_numpy(bits).to(dtype)
    expect = bitpack_oracle.bit_spike_compress(bits)
    assert np.array_equal(expect, np.packbits(bits.astype(np.uint8), bitorder="little"))
    packed = bit_spike_compress(src.cuda())
    assert packed.dtype == torch.uint8 and packed.shape == ((n + 7) // 8,)
    assert np.array_equal(packed.cpu().numpy(), expect)
    for out_dtype in (torch.uint8, torch.float32, dtype):
        back = bit_spike_decompress(packed, (n,), dtype=out_dtype)
        assert back.dtype == out_dtype
        assert torch.equal(back.cpu(), torch.from_numpy(bits).to(out_dtype))


def test_unaligned_views_take_the_elementwise_path():
    rng = np.random.default_rng(3)
    bits = rng.random(5000) < 0.5
    base = torch.from_numpy(bits).float().cuda()
    src = base[1:]  # 4-byte offset: not 16-byte aligned
    assert src.data_ptr() % 16 != 0
    packed = bit_spike_compress(src)
    assert np.array_equal(packed.cpu().numpy(), bitpack_oracle.bit_spike_compress(bits[1:]))


def test_nonzero_semantics_match_to_bool():
    vals = torch.tensor([0.0, -0.0, 1.0, 2.0, float("nan"), 1e-45, -1.0, 0.0, 0.5, 0.0, 0.0, 0.0, 0.0, 0.0, -0.0, 3.0])
    for dt in (torch.float32, torch.float16, torch.bfloat16):
        t = vals.to(dt)
        expect = bitpack_oracle.bit_spike_compress(t.to(torch.bool).numpy())
        assert np.array_equal(bit_spike_compress(t.cuda()).cpu().numpy(), expect)


def test_reference_round_trip_cases():
    # test/activation_based/test_checkpointing.py:275-282
    spikes = torch.tensor([[1.0, 0.0, 1.0], [0.0, 1.0, 0.0]], device="cuda")
    c = BitSpikeCompressor()
    packed = c.compress(spikes)
    assert packed.cpu().tolist() == [0b010101]
    torch.testing.assert_close(c.decompress(packed, tuple(spikes.shape)), spikes)
    # test/activation_based/test_cuda_custom_op_migration.py:179-190
    spike = (torch.arange(17) % 3 == 0).float().cuda()
    packed = c.compress(spike)
    assert packed.cpu().tolist() == [0b01001001, 0b10010010, 0]
    assert torch.equal(c.decompress(packed, spike.shape), spike)
    # CPU tensors stay on the CPU with the same bytes
    assert c.compress(spike.cpu()).tolist() == packed.cpu().tolist()


def test_if_fp16_inference_then_pack_config4_shape_reduced():
    """Config 4 at reduced batch: IF, soft reset, fp16, uniform[0,0.25) input, eval; spikes equal the
    torch backend's, the packed mask equals the oracle's bytes and unpacks to the same spikes."""
    x = seeded_rand((32, 2, 512, 14, 14), 1004, 0.25).half()
    a = neuron.IFNode(v_threshold=1.0, v_reset=None, step_mode="m").eval()
    b = neuron.IFNode(v_threshold=1.0, v_reset=None, step_mode="m", backend="hip").cuda().eval()
    with torch.no_grad():
        sa, sb = a(x), b(x.cuda())
    assert torch.equal(sb.cpu(), sa)
    rate = float(sa.float().mean())
    assert 0.05 < rate < 0.2
    packed = bit_spike_compress(sb)
    assert np.array_equal(packed.cpu().numpy(), bitpack_oracle.bit_spike_compress(sa.numpy()))
    assert torch.equal(bit_spike_decompress(packed, sb.shape, dtype=torch.float16), sb)
