"""CPU-only: libsjhip.so loads and exports every symbol include/sjhip.h declares; argument
validation that needs no device (errors are returned before any launch)."""

import ctypes
import os
import re

import pytest

from spikingjelly_amd.activation_based.hip_kernel import library as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "sjhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sjhip_[a-z_0-9]+)\s*\(", text)))


def test_header_and_binding_list_the_same_symbols():
    assert _declared_symbols() == sorted(L.EXPORTED_SYMBOLS)


def test_library_loads_and_exports_every_declared_symbol():
    lib = L.load()
    assert lib.sjhip_abi_version() == L.ABI_VERSION
    for name in _declared_symbols():
        assert hasattr(lib, name), name


def test_argument_validation_without_a_device():
    lib = L.load()
    p = L.NeuronParams(2.0, 1.0, 0.0, 2.0, 1, 0)
    rc = lib.sjhip_neuron_forward(L.NEURON_LIF, L.DTYPE_F32, ctypes.byref(p), 0, 16, 1, 1, None, 1, 1, 1, None, None)
    assert rc == -1 and b"T=0" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward(7, L.DTYPE_F32, ctypes.byref(p), 4, 16, 1, 1, None, 1, 1, 1, None, None)
    assert rc == -1 and b"neuron 7" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward(L.NEURON_LIF, L.DTYPE_U8, ctypes.byref(p), 4, 16, 1, 1, None, 1, 1, 1, None, None)
    assert rc == -1
    rc = lib.sjhip_neuron_forward(L.NEURON_LIF, L.DTYPE_F32, ctypes.byref(p), 4, 16, 1, 1, None, 1, None, None, None, None)
    assert rc == -1 and b"v_seq" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward_packed(L.NEURON_IF, L.DTYPE_F16, ctypes.byref(p), 4, 12, 1, 1, None, 1, None, 1, None)
    assert rc == -2 and b"multiple of 8" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward_packed(L.NEURON_IF, L.DTYPE_F16, ctypes.byref(p), 4, 16, 1, 1, None, None, None, 1, None)
    assert rc == -1 and b"NULL" in lib.sjhip_last_error()
    p_bad = L.NeuronParams(2.0, 1.0, 0.0, 2.0, 9, 0)
    rc = lib.sjhip_neuron_backward(L.NEURON_LIF, L.DTYPE_F32, ctypes.byref(p_bad), 4, 16, 1, None, None, 1, None, None,
                                   1, 1, None, None, None)
    assert rc == -2 and b"surrogate" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_backward(L.NEURON_PLIF, L.DTYPE_F32, ctypes.byref(p), 4, 16, 1, None, None, 1, None, None,
                                   1, 1, None, None, None)
    assert rc == -1 and b"PLIF" in lib.sjhip_last_error()
    # PLIF reads k = sigmoid(w) from device memory: every entry point refuses a call without its address
    rc = lib.sjhip_neuron_forward(L.NEURON_PLIF, L.DTYPE_F32, ctypes.byref(p), 4, 16, 16, 16, None, 16, 16, 16, None, None)
    assert rc == -1 and b"rtau_device" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward_packed(L.NEURON_PLIF, L.DTYPE_F32, ctypes.byref(p), 4, 16, 16, 16, None, 16, None, 16, None)
    assert rc == -1 and b"rtau_device" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_backward(L.NEURON_PLIF, L.DTYPE_F32, ctypes.byref(p), 4, 16, 16, None, None, 16, 16, None,
                                   16, 16, 16, 16, None)
    assert rc == -1 and b"rtau_device" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_backward_recompute(L.NEURON_PLIF, L.DTYPE_F32, ctypes.byref(p), 4, 16, 16, 16, None,
                                             16, None, None, 16, 16, 16, 16, None)
    assert rc == -1 and b"rtau_device" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_backward_static(L.NEURON_PLIF, L.DTYPE_F32, ctypes.byref(p), 4, 16, 16, None, None, 16, 16, None,
                                          16, 16, 16, None)
    assert rc == -1 and b"rtau_device" in lib.sjhip_last_error()
    # ILIF: the count limit, the threshold, the surrogate and the window are checked before anything is launched
    def ilif(levels, sg=L.SG_MULTI_LEVEL, v_th=1.0, lo=0.0, hi=4.0):
        return L.NeuronParams(2.0, v_th, 0.0, 0.0, sg, 0, 0.0, 0.0, 0.0, levels, lo, hi)

    for bad in (0.0, 2.5, 300.0, float("nan")):
        rc = lib.sjhip_neuron_forward(L.NEURON_ILIF, L.DTYPE_F32, ctypes.byref(ilif(bad)), 4, 16, 1, 1, None, 1, 1, 1, None, None)
        assert rc == -1 and b"level_max" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward(L.NEURON_ILIF, L.DTYPE_F32, ctypes.byref(ilif(4.0, v_th=0.0)), 4, 16, 1, 1, None, 1, 1, 1, None, None)
    assert rc == -1 and b"v_threshold" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward_packed(L.NEURON_ILIF, L.DTYPE_F16, ctypes.byref(ilif(4.0)), 4, 16, 1, 1, None, 1, None, 1, None)
    assert rc == -2 and b"counts" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_backward(L.NEURON_ILIF, L.DTYPE_F32, ctypes.byref(ilif(4.0, sg=1)), 4, 16, 1, None, None, 1, None, None,
                                   1, 1, None, None, None)
    assert rc == -1 and b"multi-level" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_backward(L.NEURON_ILIF, L.DTYPE_F32, ctypes.byref(ilif(4.0, lo=2.0, hi=1.0)), 4, 16, 1, None, None, 1,
                                   None, None, 1, 1, None, None, None)
    assert rc == -1 and b"window" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_backward(L.NEURON_LIF, L.DTYPE_F32, ctypes.byref(ilif(4.0)), 4, 16, 1, None, None, 1, None, None,
                                   1, 1, None, None, None)
    assert rc == -1 and b"belongs to ILIF" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_backward_recompute(L.NEURON_ILIF, L.DTYPE_F32, ctypes.byref(ilif(4.0, sg=0)), 4, 16, 1, 1, None,
                                             1, None, None, 1, 1, None, None, None)
    assert rc == -1 and b"multi-level" in lib.sjhip_last_error()
    rc = lib.sjhip_stbif_forward(L.DTYPE_U8, 0, 4, 16, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, None, None)
    assert rc == -1 and b"dtype" in lib.sjhip_last_error()
    rc = lib.sjhip_stbif_forward(L.DTYPE_F32, 0x01, 4, 16, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, None, None)
    assert rc == -1 and b"flags" in lib.sjhip_last_error()
    rc = lib.sjhip_stbif_forward(L.DTYPE_F32, 0, 4, 16, 1, 1, 1, 1, None, 1, 1, 1, 1, 1, None, None)
    assert rc == -1 and b"scalar" in lib.sjhip_last_error()
    rc = lib.sjhip_stbif_forward(L.DTYPE_F32, 0, 4, 16, 1, 1, 1, 1, 1, 1, 1, None, 1, 1, None, None)
    assert rc == -1 and b"NULL tensor" in lib.sjhip_last_error()
    rc = lib.sjhip_stbif_forward(L.DTYPE_F32, 0, 0, 16, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, None, None)
    assert rc == -1 and b"T=0" in lib.sjhip_last_error()
    aaif = lambda *a: lib.sjhip_aaif_forward(*a)
    rc = aaif(L.DTYPE_F32, 0, 4, 16, 1, 1, 1, 3, 1, 1, 4, 2, 0.0, 1, None, 1, None)
    assert rc == -1 and b"3 thresholds" in lib.sjhip_last_error()
    rc = aaif(L.DTYPE_F32, 0, 4, 16, 1, 1, 1, 1, 1, 1, 0, 2, 0.0, 1, None, 1, None)
    assert rc == -1 and b"channel_size=0" in lib.sjhip_last_error()
    rc = aaif(L.DTYPE_F32, 0, 4, 16, 1, 1, 1, 1, 1, 1, 4, 2, 0.0, 1, None, None, None)
    assert rc == -1 and b"v_seq" in lib.sjhip_last_error()
    rc = aaif(L.DTYPE_F32, L.FLAG_DECAY_INPUT, 4, 16, 1, 1, 1, 1, 1, 1, 4, 2, 0.0, 1, None, 1, None)
    assert rc == -1 and b"flags" in lib.sjhip_last_error()
    rc = aaif(L.DTYPE_F32, 0, 4, 16, 1, 1, None, 1, 1, 1, 4, 2, 0.0, 1, None, 1, None)
    assert rc == -1 and b"NULL" in lib.sjhip_last_error()
    rc = lib.sjhip_ssa_forward_packed(L.DTYPE_F32, 4, 2, 3, 5, 0.125, 1, 1, None)
    assert rc == -2 and b"multiple of 8" in lib.sjhip_last_error()
    rc = lib.sjhip_ssa_backward_packed(L.DTYPE_F32, 4, 2, 32, 196, 0.125, 1, None, 1, None)
    assert rc == -1 and b"NULL" in lib.sjhip_last_error()
    rc = lib.sjhip_ssa_forward_packed(L.DTYPE_F32, 4, 2, 128, 196, 0.125, 1, 1, None)
    assert rc == -2 and b"not supported" in lib.sjhip_last_error()
    izh = L.IzhikevichParams(2.0, 1.0, 0.0, -0.1, 0.8, 1.0, 2.0, 0.0, 0.0, 2.0, 1, 0)
    rc = lib.sjhip_izhikevich_forward(L.DTYPE_F32, ctypes.byref(izh), 4, 16, 1, 1, None, 1, None, None, 1, 1, None, None)
    assert rc == -1 and b"NULL tensor" in lib.sjhip_last_error()
    bad = L.IzhikevichParams(2.0, 1.0, 0.0, -0.1, 0.8, 1.0, 0.0, 0.0, 0.0, 2.0, 1, 0)
    rc = lib.sjhip_izhikevich_forward(L.DTYPE_F32, ctypes.byref(bad), 4, 16, 1, 1, 1, 1, None, None, 1, 1, None, None)
    assert rc == -1 and b"tau_w" in lib.sjhip_last_error()
    bad = L.IzhikevichParams(2.0, 1.0, 0.0, -0.1, 0.8, 1.0, 2.0, 0.0, 0.0, 2.0, 7, 0)
    rc = lib.sjhip_izhikevich_backward(L.DTYPE_F32, ctypes.byref(bad), 4, 16, 1, None, None, None, None, 1, 1, 1, 1, 1, None)
    assert rc == -2 and b"surrogate" in lib.sjhip_last_error()
    rc = lib.sjhip_izhikevich_backward(L.DTYPE_F32, ctypes.byref(izh), 4, 16, 1, None, None, None, None, 1, None, 1, 1, 1, None)
    assert rc == -1 and b"v_init" in lib.sjhip_last_error()
    rc = lib.sjhip_izhikevich_backward_replay(L.DTYPE_F32, ctypes.byref(izh), 4, 16, 1, 1, None, 1, None, None, None, None, 1, 1, 1, None)
    assert rc == -1 and b"NULL tensor" in lib.sjhip_last_error()
    rc = lib.sjhip_izhikevich_backward_replay(L.DTYPE_F32, ctypes.byref(izh), 4, 18, 16, 16, 16, 16, None, None, None, None, 16, 16, 16, None)
    assert rc == -2 and b"does not fit" in lib.sjhip_last_error()
    rc = lib.sjhip_izhikevich_backward_replay(L.DTYPE_F32, ctypes.byref(izh), 4, 16, 16, 16, 16, 8, None, None, None, None, 16, 16, 16, None)
    assert rc == -1 and b"aligned" in lib.sjhip_last_error()
    mp = L.NeuronParams(2.0, 1.0, 0.0, 2.0, 1, 0)
    rc = lib.sjhip_neuron_forward_mp(L.NEURON_LIF, L.DTYPE_F16, L.DTYPE_BF16, ctypes.byref(mp), 4, 64, 16, 16, None, 16, 16, None, None, None)
    assert rc == -1 and b"8-bit float" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward_mp(L.NEURON_QIF, L.DTYPE_F8E4M3, L.DTYPE_BF16, ctypes.byref(mp), 4, 64, 16, 16, None, 16, 16, None, None, None)
    assert rc == -2 and b"IF, LIF and PLIF only" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward_mp(L.NEURON_LIF, L.DTYPE_F8E4M3, L.DTYPE_U8, ctypes.byref(mp), 4, 64, 16, 16, None, 16, 16, None, None, None)
    assert rc == -1 and b"spike dtype" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward_mp(L.NEURON_LIF, L.DTYPE_F8E5M2, L.DTYPE_BF16, ctypes.byref(mp), 4, 66, 16, 16, None, 16, 16, None, None, None)
    assert rc == -2 and b"multiple of 4" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward_mp(L.NEURON_LIF, L.DTYPE_F8E5M2, L.DTYPE_BF16, ctypes.byref(mp), 4, 64, 16, 16, None, 8, 16, None, None, None)
    assert rc == -1 and b"aligned" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_forward_mp(L.NEURON_PLIF, L.DTYPE_F8E5M2, L.DTYPE_BF16, ctypes.byref(mp), 4, 64, 16, 16, None, 16, 16, None, None, None)
    assert rc == -1 and b"rtau_device" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_backward_mp(L.NEURON_PLIF, L.DTYPE_F8E4M3, L.DTYPE_F32, ctypes.byref(mp), 4, 64, 16, None, None, 16, 16, 16, 16, 16, 16, None, None)
    assert rc == -1 and b"workspace" in lib.sjhip_last_error()
    rc = lib.sjhip_neuron_backward_mp(L.NEURON_IF, L.DTYPE_F8E4M3, L.DTYPE_F32, ctypes.byref(mp), 4, 64, None, None, None, 16, None, None, 16, 16, None, None, None)
    assert rc == -1 and b"NULL tensor" in lib.sjhip_last_error()
    assert lib.sjhip_bit_pack(L.DTYPE_F32, -1, 1, 1, None) == -1
    assert lib.sjhip_bit_pack(L.DTYPE_F32, 0, None, None, None) == 0
    assert lib.sjhip_plif_workspace_floats(L.DTYPE_F32, 1 << 20) >= (1 << 20) // 1024
    assert lib.sjhip_set_tuning(b"fwd_block", 100) == -1
    assert lib.sjhip_set_tuning(b"fwd_block", 512) == -1  # above the kernels' launch bound
    assert lib.sjhip_set_tuning(b"fwd_block", 64) == 0 and lib.sjhip_get_tuning(b"fwd_block") == 64
    assert lib.sjhip_set_tuning(b"fwd_block", 128) == 0
    assert lib.sjhip_set_tuning(b"bwd_blocks_per_cu", 65) == -1
    assert lib.sjhip_get_tuning(b"bwd_blocks_per_cu") == 2
    assert lib.sjhip_get_tuning(b"column_spread") == 2
    assert lib.sjhip_set_tuning(b"column_spread", 3) == -1 and lib.sjhip_set_tuning(b"column_spread", -1) == -1
    assert lib.sjhip_set_tuning(b"column_spread", 65537) == -1
    assert lib.sjhip_set_tuning(b"column_spread", 256) == 0 and lib.sjhip_get_tuning(b"column_spread") == 256
    assert lib.sjhip_set_tuning(b"column_spread", 1) == 0 and lib.sjhip_get_tuning(b"column_spread") == 1
    assert lib.sjhip_set_tuning(b"column_spread", 2) == 0
    assert lib.sjhip_set_tuning(b"nope", 1) == -1


def test_python_binding_raises_with_library_message():
    with pytest.raises(RuntimeError, match="set_tuning"):
        L.set_tuning("fwd_block", 3)
    with pytest.raises(NotImplementedError):
        import torch

        L.dtype_id(torch.float64)


def test_replay_policy_follows_the_lds_footprint():
    lib = L.load()
    N = 1 << 20
    assert lib.sjhip_recompute_supported(L.DTYPE_F32, 128, N) == 1
    assert lib.sjhip_recompute_preferred(L.DTYPE_F32, 16, N, 0) == 1
    assert lib.sjhip_recompute_preferred(L.DTYPE_F32, 39, N, 0) == 1 and lib.sjhip_recompute_preferred(L.DTYPE_F32, 40, N, 0) == 0
    assert lib.sjhip_recompute_preferred(L.DTYPE_F32, 16, N + 1, 0) == 0  # not supported at all: N % 4
    # 16-bit storage has the fp32 footprint per work-item: eight neurons parked as 16-bit patterns (every op rounded)
    # or four neurons parked as fp32 (fp32 state)
    for flags in (0, L.FLAG_FP32_STATE):
        assert lib.sjhip_recompute_preferred(L.DTYPE_BF16, 39, N, flags) == 1
        assert lib.sjhip_recompute_preferred(L.DTYPE_BF16, 40, N, flags) == 0


def test_traceable_replay_policy_mirrors_the_library():
    """The functionals decide about the replay backward with integer arithmetic on limits probed from the library
    (a tracing compiler cannot follow a ctypes call): both must agree for every shape."""
    import torch

    from spikingjelly_amd.activation_based.functional import neuron as F

    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        for flags in (0, L.FLAG_FP32_STATE, L.FLAG_FP32_STATE | L.FLAG_RECIPROCAL_TAU):
            width, steps = F._replay_limits(dtype, flags)
            assert width in (4, 8) and steps == 39
            for T in (1, 8, 39, 40, 64, 159, 160, 1000):
                for N in (1, 4, 8, 12, 37, 64, 100, 4096):
                    assert (N % width == 0 and T <= steps) == L.recompute_preferred(dtype, T, N, flags), (dtype, flags, T, N)


def test_convolution_statistics_arguments_without_a_device():
    lib = L.load()
    # two partial rows per 128 columns of all samples: 256 * 196 columns -> 392 column blocks
    assert lib.sjhip_pwconv_gemm_stats_rows(384, 256, 196) == 784
    assert lib.sjhip_pwconv_gemm_stats_rows(3, 1, 4) == 2
    assert lib.sjhip_pwconv_gemm_stats_rows(0, 1, 4) == 0
    rc = lib.sjhip_pwconv_gemm_stats(16, 3, 8, 8, 16, 3, 1, 4, 16, None, None)
    assert rc == -1 and b"NULL" in lib.sjhip_last_error()
    rc = lib.sjhip_pwconv_gemm_stats(16, 3, 8, 0, 16, 3, 1, 4, 16, 16, None)
    assert rc == -1 and b"K=0" in lib.sjhip_last_error()
    rc = lib.sjhip_bn_finalize_rows(None, 4, 16, 8, None, None, 1e-5, 0.1, None, None, 16, 16, 16, 16, None, None)
    assert rc == -1 and b"NULL" in lib.sjhip_last_error()
    rc = lib.sjhip_bn_finalize_rows(16, 0, 16, 8, None, None, 1e-5, 0.1, None, None, 16, 16, 16, 16, None, None)
    assert rc == -1 and b"rows=0" in lib.sjhip_last_error()


def test_fp16_split_convolution_arguments_without_a_device():
    """The fp16 GEMM entry points refuse what they cannot run before anything is launched: bf16 entry points given fp16
    term codes, activation terms other than 1 or 2, two terms without the scale of their tensor."""
    lib = L.load()
    rc = lib.sjhip_pwconv_gemm(16, 18, 8, 8, 16, 2, 1, 4, 16, None)
    assert rc == -2 and b"sjhip_pwconv_gemm_f16" in lib.sjhip_last_error()
    rc = lib.sjhip_pwconv_grad_weight(16, 18, 16, 2, 1, 8, 8, 4, 16, 16, None)
    assert rc == -2 and b"bf16" in lib.sjhip_last_error()
    rc = lib.sjhip_pwconv_gemm_f16(16, 8, 8, 16, 3, 16, 1, 4, 16, None, None)
    assert rc == -2 and b"1 or 2" in lib.sjhip_last_error()
    rc = lib.sjhip_pwconv_gemm_f16(16, 8, 8, 16, 2, None, 1, 4, 16, None, None)
    assert rc == -1 and b"sjhip_pwconv_amax" in lib.sjhip_last_error()
    rc = lib.sjhip_pwconv_gemm_f16(None, 8, 8, 16, 1, None, 1, 4, 16, None, None)
    assert rc == -1 and b"NULL" in lib.sjhip_last_error()
    rc = lib.sjhip_pwconv_grad_weight_f16(16, None, 16, 1, None, 1, 8, 8, 4, 16, 16, None)
    assert rc == -1 and b"NULL" in lib.sjhip_last_error()
    rc = lib.sjhip_pwconv_grad_weight_f16(16, 16, 16, 2, None, 1, 8, 8, 4, 16, 16, None)
    assert rc == -1 and b"sjhip_pwconv_amax" in lib.sjhip_last_error()
    rc = lib.sjhip_pwconv_gemm_f16(16, 8, 8, 16, 2, 20, 1, 4, 16, None, None)
    assert rc == -2 and b"16-byte aligned" in lib.sjhip_last_error()
    rc = lib.sjhip_pwconv_grad_weight_f16_bits(16, 20, 16, 1, 8, 8, 4, 16, 16, None)
    assert rc == -2 and b"16-byte aligned" in lib.sjhip_last_error()
    rc = lib.sjhip_pwconv_amax(16, 0, 4, 16, None)
    assert rc == -1 and b"S=0" in lib.sjhip_last_error()
    assert lib.sjhip_pwconv_amax_floats(10) == 256 + 16 * 10
    rc = lib.sjhip_pwconv_split_weight_f16(16, 8, 8, 0, 8, None, 0, None)
    assert rc == -2 and b"aligned" in lib.sjhip_last_error()
