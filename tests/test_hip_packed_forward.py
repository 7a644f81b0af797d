"""Inference forward with bit-packed spike output against the oracle.

The packed bytes must equal ``pack(oracle spikes)`` bit for bit (so also the dense HIP forward followed by
``bit_spike_compress``), and v_seq / v_last must be the dense kernel's.
"""

import math

import numpy as np
import pytest
import torch

from oracle import bitpack_oracle
from oracle import neuron_oracle as no
from spikingjelly_amd import configure
from spikingjelly_amd.activation_based import functional
from spikingjelly_amd.activation_based.hip_kernel.compress import bit_spike_compress, bit_spike_decompress

from helpers import bits_equal, seeded_rand, seeded_randn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    from spikingjelly_amd.activation_based.hip_kernel import library, neuron_kernel

    library.load()
    return neuron_kernel


def _packed(K, kind, xd, vd, p, decay_input, vth, v_reset, store_v_seq=True, flags=0):
    soft = v_reset is None
    vr = 0.0 if soft else v_reset
    if kind == "if":
        return K.hip_multistep_if_inference_packed(xd, vd, vth, vr, soft, store_v_seq, flags)
    if kind == "lif":
        return K.hip_multistep_lif_inference_packed(xd, vd, vth, vr, soft, p, decay_input, store_v_seq, flags)
    kd = torch.as_tensor(p, dtype=torch.float32).cuda()
    return K.hip_multistep_plif_inference_packed(xd, vd, kd, vth, vr, soft, decay_input, store_v_seq, flags)


def _dense(K, kind, xd, vd, p, decay_input, vth, v_reset, store_v_seq=True, flags=0):
    soft = v_reset is None
    vr = 0.0 if soft else v_reset
    if kind == "if":
        return K.hip_multistep_if_inference(xd, vd, vth, vr, soft, store_v_seq, flags)
    if kind == "lif":
        return K.hip_multistep_lif_inference(xd, vd, vth, vr, soft, p, decay_input, store_v_seq, flags)
    kd = torch.as_tensor(p, dtype=torch.float32).cuda()
    return K.hip_multistep_plif_inference(xd, vd, kd, vth, vr, soft, decay_input, store_v_seq, flags)


GRID = [("if", None, True, 2.0), ("if", 0.0, True, 2.0), ("lif", 0.0, True, 2.0), ("lif", None, False, 3.0),
        ("lif", -0.2, True, 10.0), ("plif", None, True, 2.0), ("plif", 0.0, False, 3.0)]


@pytest.mark.parametrize("kind,v_reset,decay_input,tau", GRID)
@pytest.mark.parametrize("T,N", [(16, 8192), (5, 8), (3, 16), (7, 72), (33, 1000), (1, 64), (4, 4104)])
def test_packed_forward_fp32_equals_oracle(K, kind, v_reset, decay_input, tau, T, N):
    x = seeded_randn((T, N), 300 + T, 0.4, 1.0)
    v0 = seeded_randn((N,), 400 + N, 0.0, 0.3)
    vth = 0.8
    if kind == "plif":
        w = torch.tensor(-math.log(tau - 1.0))
        es, ev, _ = no.multi_step("plif", x, v0, w, decay_input, vth, v_reset)
        p = float(w.sigmoid())
    else:
        es, ev, _ = no.multi_step(kind, x, v0, tau, decay_input, vth, v_reset)
        p = tau
    expect = bitpack_oracle.bit_spike_compress(es.numpy().astype(bool))
    bits, v_seq, v_last = _packed(K, kind, x.cuda(), v0.cuda(), p, decay_input, vth, v_reset)
    assert bits.dtype == torch.uint8 and bits.shape == (T * N // 8,)
    assert np.array_equal(bits.cpu().numpy(), expect)
    assert bits_equal(v_seq.cpu(), ev)
    assert bits_equal(v_last.cpu(), ev[-1])
    # without v_seq
    bits2, empty, v_last2 = _packed(K, kind, x.cuda(), v0.cuda(), p, decay_input, vth, v_reset, store_v_seq=False)
    assert empty.numel() == 0
    assert torch.equal(bits2, bits) and bits_equal(v_last2.cpu(), ev[-1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("fp32_state", [False, True])
@pytest.mark.parametrize("kind,v_reset,decay_input,tau", GRID)
@pytest.mark.parametrize("T,N", [(8, 4096), (3, 8), (6, 136)])
def test_packed_forward_16bit_equals_dense_kernel_and_oracle(K, dtype, fp32_state, kind, v_reset, decay_input, tau, T, N):
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    flags = L.FLAG_FP32_STATE if fp32_state else 0
    x = seeded_randn((T, N), 500 + T, 0.4, 1.0).to(dtype)
    v0 = seeded_randn((N,), 600 + N, 0.0, 0.3).to(dtype)
    vth = 0.75
    p = float(torch.tensor(-math.log(tau - 1.0)).sigmoid()) if kind == "plif" else tau
    bits, v_seq, v_last = _packed(K, kind, x.cuda(), v0.cuda(), p, decay_input, vth, v_reset, flags=flags)
    s, dv_seq, dv_last = _dense(K, kind, x.cuda(), v0.cuda(), p, decay_input, vth, v_reset, flags=flags)
    assert torch.equal(bits, bit_spike_compress(s))
    assert bits_equal(v_seq, dv_seq) and bits_equal(v_last, dv_last)
    # against the oracle's spikes where the oracle states the same arithmetic: IF, or k = 1/2 exactly
    if fp32_state and (kind == "if" or tau == 2.0):
        es = no.multi_step_mixed_precision(kind, x, v0, dtype, 0.5, decay_input, vth, v_reset)[0]
    elif not fp32_state and kind != "plif":
        es = no.multi_step(kind, x, v0, tau, decay_input, vth, v_reset)[0]
    else:
        return  # the dense-kernel comparison above covers these; the dense kernel has its own oracle tests
    assert np.array_equal(bits.cpu().numpy(), bitpack_oracle.bit_spike_compress(es.float().numpy().astype(bool)))


def test_unaligned_tensors_take_the_elementwise_path(K):
    """A 4-byte offset makes 16-byte accesses impossible: the ballot path writes the bytes."""
    T, N = 9, 200
    flat = seeded_randn((T * N + 1,), 71, 0.4, 1.0).cuda()
    x = flat[1:].view(T, N)
    assert x.data_ptr() % 16 != 0 and x.is_contiguous()
    v0 = torch.zeros(N, device="cuda")
    es, ev, _ = no.multi_step("lif", x.cpu(), v0.cpu(), 2.0, True, 1.0, 0.0)
    bits, v_seq, v_last = _packed(K, "lif", x, v0, 2.0, True, 1.0, 0.0)
    assert np.array_equal(bits.cpu().numpy(), bitpack_oracle.bit_spike_compress(es.numpy().astype(bool)))
    assert bits_equal(v_seq.cpu(), ev)


def test_rows_that_do_not_start_on_a_byte_are_refused_by_the_kernel_and_served_by_two_kernels(K):
    x = seeded_randn((4, 12), 5, 0.5, 1.0).cuda()
    v0 = torch.zeros(12, device="cuda")
    with pytest.raises(NotImplementedError, match="N % 8"):
        K.hip_multistep_if_inference_packed(x, v0, 1.0, 0.0, True, False, 0)
    bits, v_next, v_seq = functional.if_multi_step_hip_packed(x, v0, 1.0, None)
    es, ev, _ = no.multi_step("if", x.cpu(), v0.cpu(), None, True, 1.0, None)
    assert np.array_equal(bits.cpu().numpy(), bitpack_oracle.bit_spike_compress(es.numpy().astype(bool)))
    assert v_seq is None and bits_equal(v_next.cpu(), ev[-1])


def test_functionals_round_trip_config4_reduced():
    """BASELINE config 4 at reduced batch: IF, soft reset, fp16, rate-coded input; pack -> unpack is the dense
    spike tensor, and the spike count obeys the rate-coding identity count = floor(T x) for dyadic inputs."""
    T, shape = 32, (2, 64, 14, 14)
    configure.hip_half_precision_mode = "torch"
    x = (seeded_rand((T,) + shape, 1004, 0.25)).half().cuda()
    v0 = torch.zeros(shape, dtype=torch.float16, device="cuda")
    bits, v_next, v_seq = functional.if_multi_step_hip_packed(x, v0, 1.0, None)
    s, v_next_d, _ = functional.if_multi_step_hip(x, v0, 1.0, None, None)
    back = bit_spike_decompress(bits, x.shape, dtype=torch.float16)
    assert torch.equal(back, s) and bits_equal(v_next, v_next_d) and v_seq is None
    # constant dyadic input: exact in fp16, count = floor(T x)
    xc = torch.full((T, 64), 0.1875, dtype=torch.float16, device="cuda")
    bits_c, v_c, _ = functional.if_multi_step_hip_packed(xc, torch.zeros(64, dtype=torch.float16, device="cuda"), 1.0, None)
    count = bit_spike_decompress(bits_c, xc.shape, dtype=torch.float32).sum(0)
    assert torch.equal(count.cpu(), torch.full((64,), float(math.floor(T * 0.1875))))
    assert torch.equal(v_c.float().cpu(), torch.full((64,), T * 0.1875 - math.floor(T * 0.1875)))


def test_lif_and_plif_functionals():
    x = seeded_randn((6, 4, 32), 9, 0.5, 1.0).cuda()
    v0 = torch.zeros((4, 32), device="cuda")
    w = torch.tensor(-math.log(3.0 - 1.0), device="cuda")
    for fn, dense, args in ((functional.lif_multi_step_hip_packed, functional.lif_multi_step_hip, (3.0, True, 1.0, 0.0)),
                            (functional.plif_multi_step_hip_packed, functional.plif_multi_step_hip, (w, True, 1.0, None))):
        bits, v_next, v_seq = fn(x, v0, *args, store_v_seq=True)
        s, v_next_d, v_seq_d = dense(x, v0, *args, None, store_v_seq=True)
        assert torch.equal(bit_spike_decompress(bits, x.shape, dtype=torch.float32), s)
        assert bits_equal(v_next, v_next_d) and bits_equal(v_seq, v_seq_d)
