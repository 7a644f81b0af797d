"""ctypes binding of ``oracle/sj_oracle.c`` (built by ``oracle/Makefile``).  Test infrastructure only."""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_double, c_float, c_int, c_int64, c_void_p
from typing import Optional

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_DIR, "_build", "libsjoracle.so")
_lib = None

NEURON = {"if": 0, "lif": 1, "plif": 2}


def available() -> bool:
    return os.path.exists(_PATH)


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not available():
            raise OSError(f"{_PATH} not built; run `make -C oracle`")
        lib = ctypes.CDLL(_PATH)
        lib.sjo_forward_f32.restype = None
        lib.sjo_forward_f32.argtypes = [c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_float, c_int, c_float, c_float, c_int]
        lib.sjo_backward_f64.restype = None
        lib.sjo_backward_f64.argtypes = [c_int, c_int64, c_int64] + [c_void_p] * 9 + [POINTER(c_double)] + \
                                        [c_double, c_int, c_double, c_double, c_int, c_int, c_int, c_double]
        lib.sjo_bit_pack.restype = None
        lib.sjo_bit_pack.argtypes = [c_int, c_int64, c_void_p, c_void_p]
        lib.sjo_bit_unpack_u8.restype = None
        lib.sjo_bit_unpack_u8.argtypes = [c_int64, c_void_p, c_void_p]
        _lib = lib
    return _lib


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(c_void_p)


def forward_f32(kind: str, x_seq: np.ndarray, v_init: np.ndarray, tau: float = 2.0, decay_input: bool = True,
                v_threshold: float = 1.0, v_reset: Optional[float] = 0.0):
    """fp32 forward; ``tau`` is the LIF divisor or the PLIF factor k.  Returns (spike_seq, v_seq, h_seq)."""
    x = np.ascontiguousarray(x_seq, dtype=np.float32)
    T = x.shape[0]
    x2 = x.reshape(T, -1)
    N = x2.shape[1]
    v0 = np.ascontiguousarray(v_init, dtype=np.float32).reshape(-1)
    assert v0.size == N
    s = np.empty_like(x2)
    v = np.empty_like(x2)
    h = np.empty_like(x2)
    soft = v_reset is None
    load().sjo_forward_f32(NEURON[kind], T, N, _p(x2), _p(v0), _p(s), _p(v), _p(h), None,
                           np.float32(tau), int(decay_input), np.float32(v_threshold),
                           np.float32(0.0 if soft else v_reset), int(soft))
    return s.reshape(x.shape), v.reshape(x.shape), h.reshape(x.shape)


def backward_f64(kind: str, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, k: float, decay_input: bool,
                 v_threshold: float, v_reset: Optional[float], detach_reset: bool, sg_id: int, alpha: float,
                 x_seq=None, v_init=None, v_seq=None):
    """float64 BPTT from fp32 inputs.  Returns (grad_x, grad_v_init, grad_k or None)."""
    f32 = lambda a: None if a is None else np.ascontiguousarray(a, dtype=np.float32)
    h = f32(h_seq)
    T = h.shape[0]
    h2 = h.reshape(T, -1)
    N = h2.shape[1]
    gs, gv, gl, x, v0, vs = (f32(grad_spike_seq), f32(grad_v_seq), f32(grad_v_last), f32(x_seq), f32(v_init),
                             f32(v_seq))
    gx = np.empty((T, N), dtype=np.float64)
    gvi = np.empty((N,), dtype=np.float64)
    gk = c_double(0.0)
    soft = v_reset is None
    plif = kind == "plif"
    load().sjo_backward_f64(NEURON[kind], T, N, _p(gs), _p(gv), _p(gl), _p(h2), _p(x), _p(v0), _p(vs), _p(gx),
                            _p(gvi), ctypes.byref(gk) if plif else None, float(k), int(decay_input),
                            float(v_threshold), float(0.0 if soft else v_reset), int(soft), int(detach_reset),
                            int(sg_id), float(alpha))
    return gx.reshape(h.shape), gvi.reshape(h.shape[1:]), (gk.value if plif else None)


def bit_pack(src: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(src).reshape(-1)
    if a.dtype == np.bool_:
        a = a.view(np.uint8)
    esize = a.dtype.itemsize
    assert esize in (1, 2, 4)
    out = np.empty((a.size + 7) // 8, dtype=np.uint8)
    load().sjo_bit_pack(esize, a.size, _p(a), _p(out))
    return out


def bit_unpack(packed: np.ndarray, n: int) -> np.ndarray:
    p = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty(n, dtype=np.uint8)
    load().sjo_bit_unpack_u8(n, _p(p), _p(out))
    return out
