"""ctypes binding of the C ABI declared in ``include/sjhip.h``.

The shared library is looked up next to the package (``spikingjelly_amd/libsjhip.so``,
built in-tree by ``make -C spikingjelly_amd/csrc``).  Nothing here falls back to another
implementation: a missing library raises, a failing call raises with the library's message.
"""

from __future__ import annotations

import ctypes
import os
import threading
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_int32, c_int64, c_uint32, c_void_p

import torch

ABI_VERSION = 7

# enums of include/sjhip.h
NEURON_IF, NEURON_LIF, NEURON_PLIF, NEURON_QIF, NEURON_ILIF, NEURON_EIF = 0, 1, 2, 3, 4, 5
SG_MULTI_LEVEL = 7  # ILIF's windowed straight-through estimator; ids 0-6 are listed in surrogate_registry
DTYPE_F32, DTYPE_F16, DTYPE_BF16, DTYPE_U8 = 0, 1, 2, 3
DTYPE_F8E4M3, DTYPE_F8E5M2 = 4, 5  # storage dtypes of the mixed-precision entry points only
FLAG_DECAY_INPUT = 0x01
FLAG_SOFT_RESET = 0x02
FLAG_DETACH_RESET = 0x04
FLAG_FP32_STATE = 0x10
FLAG_RECIPROCAL_TAU = 0x20
FLAG_ATOMIC_REDUCE = 0x80
FLAG_V_INIT_BROADCAST = 0x100
FLAG_Q_BROADCAST = 0x200
FLAG_ACC_BROADCAST = 0x400
FLAG_W_INIT_BROADCAST = 0x800
FLAG_GRAD_STORAGE = 0x1000
STATIC_WORKSPACE_MAX_NEURONS = 1 << 26

(KC_FORWARD, KC_BACKWARD, KC_PLIF_REDUCE, KC_BIT_PACK, KC_BIT_UNPACK, KC_SSA_FORWARD, KC_SSA_BACKWARD, KC_PW_GEMM,
 KC_PW_GRAD_WEIGHT, KC_BN_STATS, KC_BN_LIF_FORWARD, KC_BN_LIF_BACKWARD, KC_BN_GRAD_INPUT, KC_STREAM_PROBE,
 KC_MFMA_PROBE) = range(15)

EXPORTED_SYMBOLS = (
    "sjhip_abi_version",
    "sjhip_last_error",
    "sjhip_neuron_forward",
    "sjhip_neuron_forward_packed",
    "sjhip_plif_workspace_floats",
    "sjhip_neuron_forward_mp",
    "sjhip_neuron_backward_mp",
    "sjhip_neuron_backward",
    "sjhip_neuron_backward_static",
    "sjhip_neuron_backward_recompute",
    "sjhip_replay_pieces",
    "sjhip_neuron_forward_pieces",
    "sjhip_neuron_backward_recompute_pieces",
    "sjhip_recompute_supported",
    "sjhip_recompute_preferred",
    "sjhip_ssa_supported",
    "sjhip_ssa_forward",
    "sjhip_ssa_backward",
    "sjhip_ssa_forward_packed",
    "sjhip_ssa_backward_packed",
    "sjhip_ssa_lif_forward_packed",
    "sjhip_ssa_lif_backward_packed",
    "sjhip_stbif_forward",
    "sjhip_aaif_forward",
    "sjhip_izhikevich_forward",
    "sjhip_izhikevich_backward",
    "sjhip_izhikevich_backward_replay",
    "sjhip_stream_probe",
    "sjhip_mfma_probe_blocks",
    "sjhip_mfma_probe",
    "sjhip_pwconv_planes_elems",
    "sjhip_pwconv_split_weight",
    "sjhip_pwconv_gemm",
    "sjhip_pwconv_gemm_stats_rows",
    "sjhip_pwconv_gemm_stats",
    "sjhip_pwconv_grad_weight_workspace_floats",
    "sjhip_pwconv_grad_weight",
    "sjhip_pwconv_split_weight_f16",
    "sjhip_pwconv_amax",
    "sjhip_pwconv_amax_floats",
    "sjhip_pwconv_gemm_f16",
    "sjhip_pwconv_grad_weight_f16",
    "sjhip_bn_grad_input_amax",
    "sjhip_pwconv_gemm_f16_bits",
    "sjhip_pwconv_grad_weight_f16_bits",
    "sjhip_pwconv_plane_elems",
    "sjhip_pwconv_split_planes",
    "sjhip_pwconv_gemm_planes_stats_rows",
    "sjhip_pwconv_gemm_planes",
    "sjhip_pwconv_grad_weight_planes_workspace_floats",
    "sjhip_pwconv_grad_weight_planes",
    "sjhip_bn_stats",
    "sjhip_bn_finalize",
    "sjhip_bn_finalize_rows",
    "sjhip_bn_lif_forward",
    "sjhip_bn_lif_backward",
    "sjhip_bn_plif_forward",
    "sjhip_bn_plif_backward_workspace_floats",
    "sjhip_bn_plif_backward",
    "sjhip_bn_backward_finalize",
    "sjhip_bn_grad_input",
    "sjhip_bit_pack",
    "sjhip_bit_unpack",
    "sjhip_set_tuning",
    "sjhip_get_tuning",
    "sjhip_profile_enable",
    "sjhip_profile_reset",
    "sjhip_profile_read",
)


class NeuronParams(ctypes.Structure):
    """``struct sjhip_neuron_params``."""

    _fields_ = [
        ("tau", c_float),
        ("v_threshold", c_float),
        ("v_reset", c_float),
        ("sg_alpha", c_float),
        ("sg_id", c_int32),
        ("flags", c_uint32),
        ("v_rest", c_float),
        ("v_c", c_float),
        ("a0", c_float),
        ("level_max", c_float),
        ("grad_min", c_float),
        ("grad_max", c_float),
    ]


class IzhikevichParams(ctypes.Structure):
    """``struct sjhip_izhikevich_params``."""

    _fields_ = [(name, c_float) for name in ("tau", "v_threshold", "v_reset", "v_rest", "v_c", "a0", "tau_w", "a", "b",
                                             "sg_alpha")] + [("sg_id", c_int32), ("flags", c_uint32)]


_lock = threading.Lock()
_lib = None


def library_path() -> str:
    return os.path.join(os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))), "libsjhip.so")


def load() -> ctypes.CDLL:
    """Load (once) and return the library; ``OSError`` if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = library_path()
        if not os.path.exists(path):
            raise OSError(f"{path} not found; run `make -C spikingjelly_amd/csrc`")
        lib = ctypes.CDLL(path)
        lib.sjhip_abi_version.restype = c_int
        lib.sjhip_abi_version.argtypes = []
        if lib.sjhip_abi_version() != ABI_VERSION:
            raise OSError(f"{path}: ABI version {lib.sjhip_abi_version()} != {ABI_VERSION}")
        lib.sjhip_last_error.restype = c_char_p
        lib.sjhip_last_error.argtypes = []
        lib.sjhip_neuron_forward.restype = c_int
        lib.sjhip_neuron_forward.argtypes = [
            c_int, c_int, POINTER(NeuronParams), c_int64, c_int64,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        ]
        lib.sjhip_neuron_forward_packed.restype = c_int
        lib.sjhip_neuron_forward_packed.argtypes = [
            c_int, c_int, POINTER(NeuronParams), c_int64, c_int64,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        ]
        lib.sjhip_neuron_forward_mp.restype = c_int
        lib.sjhip_neuron_forward_mp.argtypes = [c_int, c_int, c_int, POINTER(NeuronParams), c_int64, c_int64] + [c_void_p] * 8
        lib.sjhip_neuron_backward_mp.restype = c_int
        lib.sjhip_neuron_backward_mp.argtypes = [c_int, c_int, c_int, POINTER(NeuronParams), c_int64, c_int64] + [c_void_p] * 11
        lib.sjhip_plif_workspace_floats.restype = c_int64
        lib.sjhip_plif_workspace_floats.argtypes = [c_int, c_int64]
        lib.sjhip_neuron_backward.restype = c_int
        lib.sjhip_neuron_backward.argtypes = [
            c_int, c_int, POINTER(NeuronParams), c_int64, c_int64,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        ]
        lib.sjhip_neuron_backward_static.restype = c_int
        lib.sjhip_neuron_backward_static.argtypes = [
            c_int, c_int, POINTER(NeuronParams), c_int64, c_int64,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
            c_void_p, c_void_p, c_void_p, c_void_p,
        ]
        lib.sjhip_neuron_backward_recompute.restype = c_int
        lib.sjhip_neuron_backward_recompute.argtypes = [
            c_int, c_int, POINTER(NeuronParams), c_int64, c_int64,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        ]
        lib.sjhip_replay_pieces.restype = c_int64
        lib.sjhip_replay_pieces.argtypes = [c_int64, c_int64]
        lib.sjhip_neuron_forward_pieces.restype = c_int
        lib.sjhip_neuron_forward_pieces.argtypes = [
            c_int, c_int, POINTER(NeuronParams), c_int64, c_int64, c_int64,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        ]
        lib.sjhip_neuron_backward_recompute_pieces.restype = c_int
        lib.sjhip_neuron_backward_recompute_pieces.argtypes = [
            c_int, c_int, POINTER(NeuronParams), c_int64, c_int64, c_int64,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        ]
        lib.sjhip_recompute_supported.restype = c_int
        lib.sjhip_recompute_supported.argtypes = [c_int, c_int64, c_int64]
        lib.sjhip_recompute_preferred.restype = c_int
        lib.sjhip_recompute_preferred.argtypes = [c_int, c_int64, c_int64, c_uint32]
        lib.sjhip_ssa_supported.restype = c_int
        lib.sjhip_ssa_supported.argtypes = [c_int, c_int, c_int64]
        lib.sjhip_ssa_forward.restype = c_int
        lib.sjhip_ssa_forward.argtypes = [c_int, c_int64, c_int, c_int, c_int64, c_float, c_void_p, c_void_p, c_void_p]
        lib.sjhip_ssa_backward.restype = c_int
        lib.sjhip_ssa_backward.argtypes = [c_int, c_int64, c_int, c_int, c_int64, c_float, c_void_p, c_void_p, c_void_p,
                                           c_void_p]
        lib.sjhip_stbif_forward.restype = c_int
        lib.sjhip_stbif_forward.argtypes = [
            c_int, c_uint32, c_int64, c_int64,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        ]
        lib.sjhip_aaif_forward.restype = c_int
        lib.sjhip_aaif_forward.argtypes = [
            c_int, c_uint32, c_int64, c_int64, c_void_p, c_void_p,
            c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_float,
            c_void_p, c_void_p, c_void_p, c_void_p,
        ]
        lib.sjhip_ssa_forward_packed.restype = c_int
        lib.sjhip_ssa_forward_packed.argtypes = [c_int, c_int64, c_int, c_int, c_int64, c_float, c_void_p, c_void_p,
                                                 c_void_p]
        lib.sjhip_ssa_backward_packed.restype = c_int
        lib.sjhip_ssa_backward_packed.argtypes = [c_int, c_int64, c_int, c_int, c_int64, c_float, c_void_p, c_void_p,
                                                  c_void_p, c_void_p]
        lib.sjhip_izhikevich_forward.restype = c_int
        lib.sjhip_izhikevich_forward.argtypes = [c_int, POINTER(IzhikevichParams), c_int64, c_int64] + [c_void_p] * 10
        lib.sjhip_izhikevich_backward.restype = c_int
        lib.sjhip_izhikevich_backward.argtypes = [c_int, POINTER(IzhikevichParams), c_int64, c_int64] + [c_void_p] * 11
        lib.sjhip_izhikevich_backward_replay.restype = c_int
        lib.sjhip_izhikevich_backward_replay.argtypes = ([c_int, POINTER(IzhikevichParams), c_int64, c_int64]
                                                         + [c_void_p] * 12)
        lib.sjhip_stream_probe.restype = c_int
        lib.sjhip_stream_probe.argtypes = [c_int, c_int, c_int, c_int64, POINTER(c_void_p), POINTER(c_void_p), c_void_p]
        lib.sjhip_mfma_probe_blocks.restype = c_int64
        lib.sjhip_mfma_probe_blocks.argtypes = [c_int]
        lib.sjhip_mfma_probe.restype = c_int
        lib.sjhip_mfma_probe.argtypes = [c_int, c_int, c_int, c_void_p, c_int64, c_void_p]
        lib.sjhip_ssa_lif_forward_packed.restype = c_int
        lib.sjhip_ssa_lif_forward_packed.argtypes = [c_int, POINTER(NeuronParams), c_int64, c_int64, c_int, c_int, c_int64, c_float] + \
                                                    [c_void_p] * 6
        lib.sjhip_ssa_lif_backward_packed.restype = c_int
        lib.sjhip_ssa_lif_backward_packed.argtypes = [c_int, POINTER(NeuronParams), c_int64, c_int64, c_int, c_int, c_int64, c_float] + \
                                                     [c_void_p] * 7
        lib.sjhip_pwconv_planes_elems.restype = c_int64
        lib.sjhip_pwconv_planes_elems.argtypes = [c_int64, c_int64]
        lib.sjhip_pwconv_split_weight.restype = c_int
        lib.sjhip_pwconv_split_weight.argtypes = [c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p]
        lib.sjhip_pwconv_gemm.restype = c_int
        lib.sjhip_pwconv_gemm.argtypes = [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64, c_int64, c_void_p,
                                          c_void_p]
        lib.sjhip_pwconv_gemm_stats_rows.restype = c_int64
        lib.sjhip_pwconv_gemm_stats_rows.argtypes = [c_int64, c_int64, c_int64]
        lib.sjhip_pwconv_gemm_stats.restype = c_int
        lib.sjhip_pwconv_gemm_stats.argtypes = [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_int64, c_int64, c_void_p,
                                                c_void_p, c_void_p]
        lib.sjhip_pwconv_grad_weight_workspace_floats.restype = c_int64
        lib.sjhip_pwconv_grad_weight_workspace_floats.argtypes = [c_int64, c_int64, c_int64]
        lib.sjhip_pwconv_grad_weight.restype = c_int
        lib.sjhip_pwconv_grad_weight.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64,
                                                 c_void_p, c_void_p, c_void_p]
        lib.sjhip_pwconv_split_weight_f16.restype = c_int
        lib.sjhip_pwconv_split_weight_f16.argtypes = [c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p, c_int64, c_void_p]
        lib.sjhip_pwconv_amax_floats.restype = c_int64
        lib.sjhip_pwconv_amax_floats.argtypes = [c_int64]
        lib.sjhip_pwconv_amax.restype = c_int
        lib.sjhip_pwconv_amax.argtypes = [c_void_p, c_int64, c_int64, c_void_p, c_void_p]
        lib.sjhip_pwconv_gemm_f16.restype = c_int
        lib.sjhip_pwconv_gemm_f16.argtypes = [c_void_p, c_int64, c_int64, c_void_p, c_int, c_void_p, c_int64, c_int64, c_void_p,
                                              c_void_p, c_void_p]
        lib.sjhip_pwconv_grad_weight_f16.restype = c_int
        lib.sjhip_pwconv_grad_weight_f16.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64,
                                                     c_int64, c_void_p, c_void_p, c_void_p]
        lib.sjhip_pwconv_gemm_f16_bits.restype = c_int
        lib.sjhip_pwconv_gemm_f16_bits.argtypes = [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p,
                                                   c_void_p]
        lib.sjhip_pwconv_grad_weight_f16_bits.restype = c_int
        lib.sjhip_pwconv_grad_weight_f16_bits.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                                          c_void_p, c_void_p, c_void_p]
        lib.sjhip_pwconv_plane_elems.restype = c_int64
        lib.sjhip_pwconv_plane_elems.argtypes = [c_int64, c_int64, c_int64, c_int]
        lib.sjhip_pwconv_split_planes.restype = c_int
        lib.sjhip_pwconv_split_planes.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p, c_void_p]
        lib.sjhip_pwconv_gemm_planes_stats_rows.restype = c_int64
        lib.sjhip_pwconv_gemm_planes_stats_rows.argtypes = [c_int64, c_int64]
        lib.sjhip_pwconv_gemm_planes.restype = c_int
        lib.sjhip_pwconv_gemm_planes.argtypes = [c_void_p, c_int64, c_int64, c_void_p, c_int, c_void_p, c_int64, c_int64,
                                                 c_void_p, c_void_p, c_void_p]
        lib.sjhip_pwconv_grad_weight_planes_workspace_floats.restype = c_int64
        lib.sjhip_pwconv_grad_weight_planes_workspace_floats.argtypes = [c_int64, c_int64, c_int64, c_int64]
        lib.sjhip_pwconv_grad_weight_planes.restype = c_int
        lib.sjhip_pwconv_grad_weight_planes.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64,
                                                        c_int64, c_void_p, c_void_p, c_void_p]
        lib.sjhip_bn_stats.restype = c_int
        lib.sjhip_bn_stats.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]
        lib.sjhip_bn_finalize.restype = c_int
        lib.sjhip_bn_finalize.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_float, c_float] + \
                                         [c_void_p] * 8
        lib.sjhip_bn_finalize_rows.restype = c_int
        lib.sjhip_bn_finalize_rows.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_float, c_float] + \
                                              [c_void_p] * 8
        lib.sjhip_bn_lif_forward.restype = c_int
        lib.sjhip_bn_lif_forward.argtypes = [c_int, POINTER(NeuronParams), c_int64, c_int64, c_int64, c_int64] + [c_void_p] * 8
        lib.sjhip_bn_lif_backward.restype = c_int
        lib.sjhip_bn_lif_backward.argtypes = [c_int, POINTER(NeuronParams), c_int64, c_int64, c_int64, c_int64] + [c_void_p] * 10
        lib.sjhip_bn_plif_forward.restype = c_int
        lib.sjhip_bn_plif_forward.argtypes = [POINTER(NeuronParams), c_int64, c_int64, c_int64, c_int64] + [c_void_p] * 9
        lib.sjhip_bn_plif_backward_workspace_floats.restype = c_int64
        lib.sjhip_bn_plif_backward_workspace_floats.argtypes = [c_int64, c_int64, c_int64]
        lib.sjhip_bn_plif_backward.restype = c_int
        lib.sjhip_bn_plif_backward.argtypes = [POINTER(NeuronParams), c_int64, c_int64, c_int64, c_int64] + [c_void_p] * 13
        lib.sjhip_bn_backward_finalize.restype = c_int
        lib.sjhip_bn_backward_finalize.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int] + [c_void_p] * 8
        lib.sjhip_bn_grad_input.restype = c_int
        lib.sjhip_bn_grad_input.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]
        lib.sjhip_bn_grad_input_amax.restype = c_int
        lib.sjhip_bn_grad_input_amax.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                                  c_void_p]
        lib.sjhip_bit_pack.restype = c_int
        lib.sjhip_bit_pack.argtypes = [c_int, c_int64, c_void_p, c_void_p, c_void_p]
        lib.sjhip_bit_unpack.restype = c_int
        lib.sjhip_bit_unpack.argtypes = [c_int, c_int64, c_void_p, c_void_p, c_void_p]
        lib.sjhip_set_tuning.restype = c_int
        lib.sjhip_set_tuning.argtypes = [c_char_p, c_int]
        lib.sjhip_get_tuning.restype = c_int
        lib.sjhip_get_tuning.argtypes = [c_char_p]
        lib.sjhip_profile_enable.restype = c_int
        lib.sjhip_profile_enable.argtypes = [c_int]
        lib.sjhip_profile_reset.restype = c_int
        lib.sjhip_profile_reset.argtypes = []
        lib.sjhip_profile_read.restype = c_int
        lib.sjhip_profile_read.argtypes = [c_int, POINTER(c_int64), POINTER(c_double)]
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().sjhip_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"libsjhip {what} failed ({rc}): {msg}")


_DTYPE_IDS = {
    torch.float32: DTYPE_F32,
    torch.float16: DTYPE_F16,
    torch.bfloat16: DTYPE_BF16,
    torch.uint8: DTYPE_U8,
    torch.bool: DTYPE_U8,
}


def dtype_id(dtype: torch.dtype, *, allow_u8: bool = False) -> int:
    """Map a torch dtype to ``sjhip_dtype``; ``NotImplementedError(dtype)`` like the
    reference kernels (cuda_kernel/neuron_kernel/multi_step/base.py:22-27)."""
    did = _DTYPE_IDS.get(dtype)
    if did is None or (did == DTYPE_U8 and not allow_u8):
        raise NotImplementedError(dtype)
    return did


def require_device_tensor(name: str, t: torch.Tensor) -> None:
    if t.device.type != "cuda":
        raise RuntimeError(
            f"backend='hip' runs on a ROCm device only, but {name} is on {t.device}; "
            "use backend='torch' for CPU tensors."
        )


def current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def ptr(t) -> int | None:
    return None if t is None else t.data_ptr()


def recompute_preferred(dtype: torch.dtype, T: int, N: int, flags: int) -> bool:
    """Whether the replay backward is supported and expected to be faster than a saved ``h_seq`` (short enough T)."""
    return bool(load().sjhip_recompute_preferred(dtype_id(dtype), T, N, flags))


def recompute_supported(dtype: torch.dtype, T: int, N: int) -> bool:
    """Whether the backward can replay the forward from ``x_seq`` instead of reading a saved ``h_seq``."""
    return bool(load().sjhip_recompute_supported(dtype_id(dtype), T, N))


def aligned16(t: torch.Tensor) -> torch.Tensor:
    """``t`` made contiguous and 16-byte aligned (a fresh allocation always is)."""
    t = t.contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()


def mfma_probe(random_operands: bool, wavefronts_per_simd: int, iterations: int, sink) -> int:
    """One launch of the matrix-core probe (see ``sjhip_mfma_probe``); returns the floating-point operations it performs.
    ``sink`` is an fp32 device tensor of at least ``sjhip_mfma_probe_blocks(wavefronts_per_simd)`` elements."""
    with torch.cuda.device(sink.device):
        rc = load().sjhip_mfma_probe(1 if random_operands else 0, wavefronts_per_simd, iterations, sink.data_ptr(), sink.numel(),
                                     current_stream_ptr(sink.device))
    check(rc, "mfma_probe")
    return load().sjhip_mfma_probe_blocks(wavefronts_per_simd) * 4 * iterations * 16 * 2 * 32 * 32 * 16


def stream_probe(reads: int, writes: int, nontemporal: bool, inputs, outputs) -> None:
    """One launch of the bandwidth probe over equally sized fp32 device tensors (see ``sjhip_stream_probe``)."""
    ref = (list(inputs) + list(outputs))[0]
    n = ref.numel()
    ins = (c_void_p * max(len(inputs), 1))(*[t.data_ptr() for t in inputs])
    outs = (c_void_p * max(len(outputs), 1))(*[t.data_ptr() for t in outputs])
    with torch.cuda.device(ref.device):
        rc = load().sjhip_stream_probe(reads, writes, 1 if nontemporal else 0, n, ins, outs, current_stream_ptr(ref.device))
    check(rc, "stream_probe")


def set_tuning(key: str, value: int) -> None:
    check(load().sjhip_set_tuning(key.encode(), int(value)), f"set_tuning({key})")


def get_tuning(key: str) -> int:
    return load().sjhip_get_tuning(key.encode())


def profile_enable(on: bool) -> None:
    check(load().sjhip_profile_enable(1 if on else 0), "profile_enable")


def profile_reset() -> None:
    check(load().sjhip_profile_reset(), "profile_reset")


def profile_read(which: int) -> tuple[int, float]:
    """(launch count, total milliseconds) of kernel class ``which`` since the last reset."""
    n = c_int64(0)
    ms = c_double(0.0)
    check(load().sjhip_profile_read(which, ctypes.byref(n), ctypes.byref(ms)), "profile_read")
    return n.value, ms.value
