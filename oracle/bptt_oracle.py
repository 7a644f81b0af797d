"""Closed-form BPTT of IF / LIF / PLIF in numpy float64.  Test infrastructure only.

Derived from the reference's kernels (``cuda_kernel/neuron_kernel/multi_step/base.py:293-409``;
LIF hooks ``lif.py:89-102``; PLIF ``plif.py:143-203``) and equal to autograd through
``functional/neuron.py:225-228, 849-852, 1290-1297``:

    sg_t   = surrogate'(h_t - v_th)         s_t = spike used in the reset branch
    dvdh_t = hard: (1 - s_t) + [not detach] (v_reset - h_t) sg_t     soft: 1 - [not detach] v_th sg_t
    G_t    = (G_{t+1} (1 - k) + grad_v_seq[t]) dvdh_t + grad_spike[t] sg_t       (G_T (1-k) := grad_v_last)
    grad_x[t] = G_t (k if decay_input else 1)        grad_v_init = G_0 (1 - k)
    PLIF: grad_k = sum G_t dh_t/dk,  dh_t/dk = x_t - (v_{t-1} - vr) (decay_input) or vr - v_{t-1}

with k = 1/tau (LIF) or sigmoid(w) (PLIF); IF uses k = 0 in (1 - k) and factor 1 for grad_x.
"""

from __future__ import annotations

from typing import Callable, Optional

import numpy as np


def bptt(kind: str, h_seq: np.ndarray, s_seq: np.ndarray, sg_prime: Callable[[np.ndarray], np.ndarray],
         grad_spike_seq: np.ndarray, grad_v_seq: Optional[np.ndarray], grad_v_last: Optional[np.ndarray],
         k: float, decay_input: bool, v_threshold: float, v_reset: Optional[float], detach_reset: bool,
         v_prev_seq: Optional[np.ndarray] = None, x_seq: Optional[np.ndarray] = None):
    """Returns (grad_x [T,N], grad_v_init [N], grad_k float or None)."""
    T = h_seq.shape[0]
    h_seq = np.asarray(h_seq, dtype=np.float64)
    s_seq = np.asarray(s_seq, dtype=np.float64)
    if kind == "if":
        kx, km = 1.0, 1.0
    else:
        kx, km = (k if decay_input else 1.0), 1.0 - k
    live = 0.0 if detach_reset else 1.0
    vr = 0.0 if v_reset is None else v_reset
    carry = np.zeros_like(h_seq[0]) if grad_v_last is None else np.asarray(grad_v_last, dtype=np.float64).copy()
    grad_x = np.zeros_like(h_seq)
    grad_k = 0.0
    for t in range(T - 1, -1, -1):
        sg = sg_prime(h_seq[t] - v_threshold)
        if v_reset is None:
            dvdh = 1.0 - live * v_threshold * sg
        else:
            dvdh = (1.0 - s_seq[t]) + live * (v_reset - h_seq[t]) * sg
        gv = carry if grad_v_seq is None else carry + grad_v_seq[t]
        G = gv * dvdh + grad_spike_seq[t] * sg
        grad_x[t] = G * kx
        carry = G * km
        if kind == "plif":
            dh_dk = (x_seq[t] - (v_prev_seq[t] - vr)) if decay_input else (vr - v_prev_seq[t])
            grad_k += float(np.sum(G * dh_dk))
    return grad_x, carry, (grad_k if kind == "plif" else None)


def bptt_ilif(h_seq: np.ndarray, grad_spike_seq: np.ndarray, grad_v_seq: Optional[np.ndarray],
              grad_v_last: Optional[np.ndarray], k: float, v_threshold: float, grad_min: float, grad_max: float,
              detach_reset: bool):
    """ILIF (``triton_kernel/neuron_kernel/ilif.py:300-326``; equal to autograd through
    ``functional/neuron.py:1097-1099`` and ``quantize.py:594-598``): with w_t = [grad_min <= h_t/v_th <= grad_max]

        G_t = Gv_t + (grad_spike[t] - [not detach] v_th Gv_t) w_t / v_th,   Gv_t = G_{t+1} (1 - k) + grad_v_seq[t]
        grad_x[t] = G_t        grad_v_init = G_0 (1 - k)

    Returns (grad_x [T,N], grad_v_init [N])."""
    h_seq = np.asarray(h_seq, dtype=np.float64)
    T = h_seq.shape[0]
    carry = np.zeros_like(h_seq[0]) if grad_v_last is None else np.asarray(grad_v_last, dtype=np.float64).copy()
    grad_x = np.zeros_like(h_seq)
    live = 0.0 if detach_reset else 1.0
    for t in range(T - 1, -1, -1):
        z = h_seq[t] / v_threshold
        w = ((z >= grad_min) & (z <= grad_max)).astype(np.float64)
        gv = carry if grad_v_seq is None else carry + grad_v_seq[t]
        G = gv + (grad_spike_seq[t] - live * v_threshold * gv) * w / v_threshold
        grad_x[t] = G
        carry = G * (1.0 - k)
    return grad_x, carry


def bptt_izhikevich(h_seq: np.ndarray, v_init: np.ndarray, sg_prime: Callable[[np.ndarray], np.ndarray],
                    grad_spike_seq: np.ndarray, grad_v_seq: Optional[np.ndarray], grad_w_seq: Optional[np.ndarray],
                    grad_v_last: Optional[np.ndarray], grad_w_last: Optional[np.ndarray], params, v_threshold: float,
                    v_reset: Optional[float], detach_reset: bool):
    """Two coupled states (equal to autograd through ``functional/neuron.py:1514-1522``); ``params`` = (tau, a0,
    v_rest, v_c, tau_w, a, b), k = 1/tau, kw = 1/tau_w:

        gv_t = grad_v_seq[t] + Gh_{t+1} (1 + k a0 ((v_t - v_c) + (v_t - v_rest)))      gw_t = grad_w_seq[t] + cw_{t+1}
        dvdh = soft: 1 - [not detach] v_th sg_t        hard: (1 - s_t) + sg_t (v_reset - [not detach] h_t)
        Gh_t = gv_t dvdh + (grad_spike[t] + b gw_t) sg_t + gw_t kw a          cw_t = gw_t (1 - kw) - Gh_t k
        grad_x[t] = Gh_t k     grad_v_init = Gh_0 (1 + k a0 (...v_init...))     grad_w_init = cw_0

    Returns (grad_x, grad_v_init, grad_w_init)."""
    tau, a0, v_rest, v_c, tau_w, a, b = params
    k, kw = 1.0 / tau, 1.0 / tau_w
    h_seq = np.asarray(h_seq, dtype=np.float64)
    T = h_seq.shape[0]
    live = 0.0 if detach_reset else 1.0
    gh = np.zeros_like(h_seq[0])
    cw = np.zeros_like(gh) if grad_w_last is None else np.asarray(grad_w_last, dtype=np.float64).copy()
    grad_x = np.zeros_like(h_seq)
    dhdv = lambda v: 1.0 + k * a0 * ((v - v_c) + (v - v_rest))
    for t in range(T - 1, -1, -1):
        h = h_seq[t]
        s = (h - v_threshold >= 0).astype(np.float64)
        v_t = h - s * v_threshold if v_reset is None else (1.0 - s) * h + s * v_reset
        sg = sg_prime(h - v_threshold)
        if t == T - 1:
            gv = np.zeros_like(h) if grad_v_last is None else np.asarray(grad_v_last, dtype=np.float64)
        else:
            gv = gh * dhdv(v_t)
        if grad_v_seq is not None:
            gv = gv + grad_v_seq[t]
        gw = cw if grad_w_seq is None else cw + grad_w_seq[t]
        dvdh = (1.0 - live * v_threshold * sg) if v_reset is None else ((1.0 - s) + sg * (v_reset - live * h))
        gh = gv * dvdh + (grad_spike_seq[t] + b * gw) * sg + gw * kw * a
        grad_x[t] = gh * k
        cw = gw * (1.0 - kw) - gh * k
    return grad_x, gh * dhdv(np.asarray(v_init, dtype=np.float64)), cw
