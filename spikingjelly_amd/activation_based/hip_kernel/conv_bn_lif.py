"""Kernel-size-1 convolution, batch normalisation and the multi-step LIF that follows them, on the hip kernels.

The block ``SeqToANNContainer(Conv1d(k=1, bias=False), BatchNorm1d) -> LIFNode`` appears twice in the reference's
``SpikingSelfAttention`` (layer/attention.py:310-329, 370-384) and, with ``Conv2d`` / ``BatchNorm2d``, in
``SpikformerConv2dBNLIF`` (model/spikformer.py:107-212); there torch runs the convolution (MIOpen / hipBLASLt, with
layout transposes around them), batch norm and the neuron as separate operators.  Here, for fp32 ``[T, B, C, L]``
tensors (``L`` the flattened positions, a multiple of 4):

* the convolution and its two gradients are GEMMs on the 16-bit matrix cores with the fp32 operands split into terms
  (``csrc/pwconv.hip``): two fp16 terms of power-of-two scaled operands (``configure.hip_conv_split = "f16"``, the
  default: three products, fp32 accuracy) or up to three bf16 terms (``"bf16"``; ``configure.hip_conv_terms`` = 3 keeps
  fp32 accuracy with six products, 2 and 1 trade it for speed); an input that is known to be spikes needs one term;
* batch norm and the neuron are two passes over the convolution output (``csrc/bn_lif.hip``): per-channel statistics,
  then normalise + charge + fire + reset over the T steps in registers, spikes written dense or bit-packed; the
  normalised tensor never exists.  The backward replays the neuron from the convolution output.

Ordinary eager calls go through ``autograd.Function`` s; under a tracing compiler (``torch.compile``) the same launch
helpers run as ``torch.library`` operators with fake kernels and registered backward formulas (``fused_ops.py``), so a
compiled module keeps the fused chain (reference: the kernel backends are compile-transparent custom operators,
``cuda_kernel/neuron_kernel/multi_step/lif.py:144-225``, ``test/activation_based/test_compile_compat.py:125-170``).

Three entries share the pieces: ``bn_lif`` (any convolution output, e.g. a 3x3 ``Conv2d`` run by torch),
``conv_bn_lif`` (the whole block) and ``conv_bn_lif_ssa`` (the block feeding the spiking self-attention contraction
through bit-packed spikes).  All are ``autograd.Function`` s around plain launch helpers; nothing here falls back to
another implementation: callers check ``supported()`` first and keep torch's operators for what it refuses.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ... import configure
from . import library as L
from . import neuron_kernel as K

__all__ = ["supported", "bn_lif", "conv_bn_lif", "conv_bn_lif_ssa", "conv_bn_lif_ssa_lif", "lif_conv_bn_lif",
           "lif_conv_bn_lif_supported", "split_weight", "pw_gemm",
           "pw_grad_weight", "pw_gemm_bits", "pw_grad_weight_bits", "amax", "F16", "split_planes", "pw_gemm_planes",
           "pw_grad_weight_planes"]

MAX_REPLAY_STEPS = 256  # the backward replays the neuron in pieces of 16 steps, one parked state per piece in LDS


F16 = 16  # term code of an fp16 operand: F16 | 2 (hi and lo of a scaled value) or F16 | 1 (exact in fp16)
_AMAX_FLOATS = 256  # SJHIP_PW_AMAX_FLOATS: the words of a tensor's largest magnitude
_AMAX_SAMPLE_WORDS = 16  # SJHIP_PW_AMAX_SAMPLE_WORDS: then so many adjacent words per sample


def amax_floats(samples: int) -> int:
    """Length of the amax buffer of a tensor of ``samples`` samples (``sjhip_pwconv_amax_floats``)."""
    return _AMAX_FLOATS + _AMAX_SAMPLE_WORDS * int(samples)


def sample_amax(words: torch.Tensor) -> torch.Tensor:
    """The largest magnitude of every sample, from the amax buffer of a tensor."""
    return words[_AMAX_FLOATS:].view(-1, _AMAX_SAMPLE_WORDS).amax(dim=1)


def _terms() -> int:
    """Term code of an operand with arbitrary fp32 values."""
    mode = getattr(configure, "hip_conv_split", "f16")
    if mode == "f16":
        return F16 | 2
    if mode != "bf16":
        raise ValueError(f"configure.hip_conv_split must be 'f16' or 'bf16', got {mode!r}")
    t = int(getattr(configure, "hip_conv_terms", 3))
    if t not in (1, 2, 3):
        raise ValueError(f"configure.hip_conv_terms must be 1, 2 or 3, got {t}")
    return t


def _exact(terms: int) -> int:
    """Term code, in the format of ``terms``, of an operand that 16-bit floats hold exactly (spikes)."""
    return (terms & F16) | 1


def supported(x_seq: torch.Tensor, need_grad: bool) -> bool:
    """fp32 device tensor ``[T, B, C, L]`` whose rows of ``L`` elements start on 16 bytes; at most ``MAX_REPLAY_STEPS`` steps when a
    backward will follow."""
    return (x_seq.is_cuda and x_seq.dtype == torch.float32 and x_seq.dim() == 4 and x_seq.shape[-1] % 4 == 0
            and x_seq.numel() > 0 and (not need_grad or x_seq.shape[0] <= MAX_REPLAY_STEPS))


def _stream(t: torch.Tensor) -> int:
    return L.current_stream_ptr(t.device)


# ------------------------------------------------------------------------------------------------
# launch helpers (no autograd)
# ------------------------------------------------------------------------------------------------
def split_weight(weight: torch.Tensor, transpose: bool, terms: int = 3, amax_reset: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Term planes of ``weight [Cout, Cin]`` (or of its transpose), the A operand of ``pw_gemm``: bf16 planes
    ``[3, rows_pad, cols_pad]``, or with ``terms & F16`` two fp16 planes of the rows scaled by powers of two, followed by
    the inverse scales (an opaque buffer either way).  ``amax_reset`` (fp16 terms): an ``amax`` buffer (of
    ``amax_floats(S)`` words) that the launch clears on the way."""
    rows, cols = weight.shape
    w = L.aligned16(weight.detach().to(torch.float32))
    planes = torch.empty(L.load().sjhip_pwconv_planes_elems(cols if transpose else rows, rows if transpose else cols),
                         dtype=torch.bfloat16, device=weight.device)
    with torch.cuda.device(weight.device):
        if terms & F16:
            reset_samples = (amax_reset.numel() - _AMAX_FLOATS) // _AMAX_SAMPLE_WORDS if amax_reset is not None else 0
            rc = L.load().sjhip_pwconv_split_weight_f16(w.data_ptr(), rows, cols, 1 if transpose else 0, planes.data_ptr(),
                                                        L.ptr(amax_reset), reset_samples, _stream(w))
        else:
            rc = L.load().sjhip_pwconv_split_weight(w.data_ptr(), rows, cols, 1 if transpose else 0, planes.data_ptr(), _stream(w))
    L.check(rc, "pwconv_split_weight")
    return planes


def amax(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The largest magnitudes in ``x [S, ...]`` as a small device buffer: the maximum of its first ``_AMAX_FLOATS`` words
    is that of the whole tensor (several words, so that the blocks that write them do not meet on one address), and
    ``sample_amax(words)[s]`` is that of sample ``s``: what the fp16 split of a tensor of arbitrary values is scaled by (the
    kernels turn it into a power of two; per sample where a GEMM's columns are samples, per tensor where it sums over
    them).  A tensor without a sample axis is one sample.  ``out``: a buffer of ``amax_floats(S)`` words that already holds
    zeros (or earlier maxima to keep)."""
    x = L.aligned16(x)
    S = x.shape[0] if x.dim() >= 2 else 1
    if out is None:
        out = torch.zeros((amax_floats(S),), dtype=torch.float32, device=x.device)
    elif out.numel() != amax_floats(S):
        raise ValueError(f"the amax buffer of {S} samples has {amax_floats(S)} words, got {out.numel()}")
    with torch.cuda.device(x.device):
        rc = L.load().sjhip_pwconv_amax(x.data_ptr(), S, x.numel() // S, out.data_ptr(), _stream(x))
    L.check(rc, "pwconv_amax")
    return out


def pw_gemm(planes: torch.Tensor, a_terms: int, M: int, Kdim: int, b: torch.Tensor, b_terms: int, stats: bool = False,
            b_amax: Optional[torch.Tensor] = None):
    """``c[s] = A b[s]`` for ``b [S, K, L]`` -> ``c [S, M, L]``.  With ``stats`` the result is ``(c, partial)``:
    ``partial [rows, M, 2]`` holds sums and sums of squares of every row of ``c`` over groups of its columns, the input
    of ``_bn_map``.  fp16 terms (``a_terms & F16``, planes from ``split_weight(..., terms)``): ``b_amax`` is
    ``amax(b)``, computed here when not given."""
    S, Kb, Lp = b.shape
    assert Kb == Kdim
    b = L.aligned16(b)
    c = torch.empty((S, M, Lp), dtype=torch.float32, device=b.device)
    lib = L.load()
    partial = None
    with torch.cuda.device(b.device):
        if stats:
            rows = lib.sjhip_pwconv_gemm_stats_rows(Kdim, S, Lp)
            partial = torch.empty((rows, M, 2), dtype=torch.float32, device=b.device)
        if a_terms & F16:
            if (a_terms & ~F16) != 2 or not b_terms & F16:
                raise ValueError(f"fp16 weight planes hold two terms and take fp16 activation terms, got {a_terms}, {b_terms}")
            if (b_terms & ~F16) == 2 and b_amax is None:
                b_amax = amax(b)
            rc = lib.sjhip_pwconv_gemm_f16(planes.data_ptr(), M, Kdim, b.data_ptr(), b_terms & ~F16, L.ptr(b_amax), S, Lp,
                                           c.data_ptr(), L.ptr(partial), _stream(b))
        elif stats:
            rc = lib.sjhip_pwconv_gemm_stats(planes.data_ptr(), a_terms, M, Kdim, b.data_ptr(), b_terms, S, Lp, c.data_ptr(),
                                             partial.data_ptr(), _stream(b))
        else:
            rc = lib.sjhip_pwconv_gemm(planes.data_ptr(), a_terms, M, Kdim, b.data_ptr(), b_terms, S, Lp, c.data_ptr(), _stream(b))
    L.check(rc, "pwconv_gemm")
    return (c, partial) if stats else c


def pw_grad_weight(dy: torch.Tensor, dy_terms: int, x: torch.Tensor, x_terms: int, dy_amax: Optional[torch.Tensor] = None,
                   x_amax: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``dw[m, n] = sum_{s, l} dy[s, m, l] x[s, n, l]``; with fp16 terms the largest magnitudes (``amax``) are computed
    here when not given."""
    S, M, Lp = dy.shape
    N = x.shape[1]
    dy, x = L.aligned16(dy), L.aligned16(x)
    lib = L.load()
    ws = torch.empty(lib.sjhip_pwconv_grad_weight_workspace_floats(M, N, S), dtype=torch.float32, device=dy.device)
    dw = torch.empty((M, N), dtype=torch.float32, device=dy.device)
    with torch.cuda.device(dy.device):
        if dy_terms & F16:
            if (dy_terms & ~F16) != 2 or not x_terms & F16:
                raise ValueError(f"the fp16 weight gradient takes two gradient terms and fp16 activation terms, got {dy_terms}, {x_terms}")
            if dy_amax is None:
                dy_amax = amax(dy)
            if (x_terms & ~F16) == 2 and x_amax is None:
                x_amax = amax(x)
            rc = lib.sjhip_pwconv_grad_weight_f16(dy.data_ptr(), dy_amax.data_ptr(), x.data_ptr(), x_terms & ~F16, L.ptr(x_amax),
                                                  S, M, N, Lp, dw.data_ptr(), ws.data_ptr(), _stream(dy))
        else:
            rc = lib.sjhip_pwconv_grad_weight(dy.data_ptr(), dy_terms, x.data_ptr(), x_terms, S, M, N, Lp, dw.data_ptr(),
                                              ws.data_ptr(), _stream(dy))
    L.check(rc, "pwconv_grad_weight")
    return dw


def pw_gemm_bits(planes: torch.Tensor, M: int, Kdim: int, bits: torch.Tensor, S: int, Lp: int, stats: bool = False):
    """``pw_gemm`` on fp16 weight planes for a spike tensor ``[S, K, L]`` that arrives bit-packed (``bits``: the byte
    array of ``bit_spike_compress`` / ``sjhip_neuron_forward_packed``); ``K * L`` a multiple of 8."""
    c = torch.empty((S, M, Lp), dtype=torch.float32, device=bits.device)
    lib = L.load()
    partial = None
    with torch.cuda.device(bits.device):
        if stats:
            partial = torch.empty((lib.sjhip_pwconv_gemm_stats_rows(Kdim, S, Lp), M, 2), dtype=torch.float32, device=bits.device)
        rc = lib.sjhip_pwconv_gemm_f16_bits(planes.data_ptr(), M, Kdim, bits.data_ptr(), S, Lp, c.data_ptr(), L.ptr(partial),
                                            _stream(bits))
    L.check(rc, "pwconv_gemm_f16_bits")
    return (c, partial) if stats else c


def pw_grad_weight_bits(dy: torch.Tensor, bits: torch.Tensor, N: int, dy_amax: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``pw_grad_weight`` with two fp16 terms of ``dy [S, M, L]`` and the spike tensor ``x [S, N, L]`` bit-packed."""
    S, M, Lp = dy.shape
    dy = L.aligned16(dy)
    lib = L.load()
    ws = torch.empty(lib.sjhip_pwconv_grad_weight_workspace_floats(M, N, S), dtype=torch.float32, device=dy.device)
    dw = torch.empty((M, N), dtype=torch.float32, device=dy.device)
    if dy_amax is None:
        dy_amax = amax(dy)
    with torch.cuda.device(dy.device):
        rc = lib.sjhip_pwconv_grad_weight_f16_bits(dy.data_ptr(), dy_amax.data_ptr(), bits.data_ptr(), S, M, N, Lp, dw.data_ptr(),
                                                   ws.data_ptr(), _stream(dy))
    L.check(rc, "pwconv_grad_weight_f16_bits")
    return dw


def split_planes(x: torch.Tensor, x_amax: Optional[torch.Tensor], terms: int = 2) -> torch.Tensor:
    """fp16 term planes of ``x [S, C, L]`` (``L`` a multiple of 4): ``terms`` planes ``[C, ld]`` with the columns
    ``s * L + l`` of all samples in a row, scaled by the power of two that ``x_amax`` (``amax(x)``) gives; one term and no
    scale for values that fp16 holds exactly.  The operand format of ``pw_gemm_planes`` / ``pw_grad_weight_planes``."""
    S, C, Lp = x.shape
    x = L.aligned16(x)
    lib = L.load()
    planes = torch.empty((lib.sjhip_pwconv_plane_elems(S, C, Lp, terms),), dtype=torch.float16, device=x.device)
    with torch.cuda.device(x.device):
        rc = lib.sjhip_pwconv_split_planes(x.data_ptr(), S, C, Lp, terms, L.ptr(x_amax), planes.data_ptr(), _stream(x))
    L.check(rc, "pwconv_split_planes")
    return planes


def pw_gemm_planes(w_planes: torch.Tensor, M: int, Kdim: int, b_planes: torch.Tensor, b_terms: int, b_amax: Optional[torch.Tensor],
                   S: int, Lp: int, stats: bool = False):
    """``pw_gemm`` on fp16 weight planes with the activations as term planes (``split_planes`` or a kernel that writes
    them): ``c [S, M, L]``, and with ``stats`` the partial batch-norm sums as well."""
    c = torch.empty((S, M, Lp), dtype=torch.float32, device=b_planes.device)
    lib = L.load()
    partial = None
    with torch.cuda.device(b_planes.device):
        if stats:
            partial = torch.empty((lib.sjhip_pwconv_gemm_planes_stats_rows(S, Lp), M, 2), dtype=torch.float32, device=c.device)
        rc = lib.sjhip_pwconv_gemm_planes(w_planes.data_ptr(), M, Kdim, b_planes.data_ptr(), b_terms, L.ptr(b_amax), S, Lp,
                                          c.data_ptr(), L.ptr(partial), _stream(c))
    L.check(rc, "pwconv_gemm_planes")
    return (c, partial) if stats else c


def pw_grad_weight_planes(dy_planes: torch.Tensor, dy_amax: torch.Tensor, x_planes: torch.Tensor, x_terms: int,
                          x_amax: Optional[torch.Tensor], S: int, M: int, N: int, Lp: int) -> torch.Tensor:
    """``dw [M, N] = sum_{s, l} dy[s, m, l] x[s, n, l]`` from the term planes of ``dy`` (two terms) and of ``x``."""
    lib = L.load()
    dev = dy_planes.device
    ws = torch.empty(lib.sjhip_pwconv_grad_weight_planes_workspace_floats(M, N, S, Lp), dtype=torch.float32, device=dev)
    dw = torch.empty((M, N), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = lib.sjhip_pwconv_grad_weight_planes(dy_planes.data_ptr(), dy_amax.data_ptr(), x_planes.data_ptr(), x_terms,
                                                 L.ptr(x_amax), S, M, N, Lp, dw.data_ptr(), ws.data_ptr(), _stream(dw))
    L.check(rc, "pwconv_grad_weight_planes")
    return dw


def _bn_map(y: torch.Tensor, gamma, beta, running_mean, running_var, batch_stats: bool, momentum: float, eps: float,
            partial: Optional[torch.Tensor] = None, tracked: Optional[torch.Tensor] = None):
    """Per-channel ``(scale, shift, mean, invstd)`` of ``z = y * scale + shift`` for ``y [S, C, L]``; with
    ``batch_stats`` from the statistics of ``y`` (and the running statistics, when given, are updated in place).
    ``partial``: the sums the convolution left behind (``pw_gemm(..., stats=True)``), which save the pass over ``y``.
    ``tracked``: the batch norm's ``num_batches_tracked`` (int64, on the device), which the same launch increments."""
    S, C, Lp = y.shape
    lib = L.load()
    out = torch.empty((4, C), dtype=torch.float32, device=y.device)
    with torch.cuda.device(y.device):
        if batch_stats and partial is not None:
            rc = lib.sjhip_bn_finalize_rows(partial.data_ptr(), partial.shape[0], S * Lp, C, L.ptr(gamma), L.ptr(beta), eps,
                                            momentum, L.ptr(running_mean), L.ptr(running_var), out[0].data_ptr(),
                                            out[1].data_ptr(), out[2].data_ptr(), out[3].data_ptr(), L.ptr(tracked), _stream(y))
            L.check(rc, "bn_finalize_rows")
            return out
        partial = None
        if batch_stats:
            partial = torch.empty((S * C, 2), dtype=torch.float32, device=y.device)
            L.check(lib.sjhip_bn_stats(y.data_ptr(), S, C, Lp, partial.data_ptr(), _stream(y)), "bn_stats")
        rc = lib.sjhip_bn_finalize(L.ptr(partial), S, C, Lp, L.ptr(gamma), L.ptr(beta), eps, momentum, L.ptr(running_mean),
                                   L.ptr(running_var), out[0].data_ptr(), out[1].data_ptr(), out[2].data_ptr(),
                                   out[3].data_ptr(), L.ptr(tracked), _stream(y))
    L.check(rc, "bn_finalize")
    return out


def _lif_params(spec, flags_extra: int = 0) -> L.NeuronParams:
    tau, v_th, v_reset, flags, sg_id, sg_alpha = spec
    return K._params(tau, v_th, v_reset, sg_alpha, sg_id, flags | flags_extra)


def _neuron_id(spec, k) -> int:
    """The neuron a spec stands for: a time constant of 0 means there is none, i.e. an IF neuron (a parametric LIF, whose
    spec carries 0 as well, brings its ``k`` as a tensor and is launched through its own entry points)."""
    return L.NEURON_IF if spec[0] == 0.0 and k is None else L.NEURON_LIF


def _bn_lif_forward(y: torch.Tensor, bn_map: torch.Tensor, v_init: torch.Tensor, spec, packed: bool,
                    k: Optional[torch.Tensor] = None):
    """``y [T, B, C, L]`` -> (spikes ``[T, B, C, L]`` fp32 or the bit-packed byte array, ``v_last [B, C, L]``).
    ``k``: one fp32 element on the device, ``sigmoid(w)`` of a parametric LIF (``spec[0]`` is then unused)."""
    T, B, C, Lp = y.shape
    v_keep, broadcast = K._state_arg(v_init, True)
    params = _lif_params(spec, broadcast)
    v_last = torch.empty((B, C, Lp), dtype=torch.float32, device=y.device)
    if packed:
        spikes = torch.empty((T * B * C * Lp // 8,), dtype=torch.uint8, device=y.device)
    else:
        spikes = torch.empty_like(y)
    k_keep, k_ptr = K._k_pointer(k, y)
    with torch.cuda.device(y.device):
        if k is None:
            rc = L.load().sjhip_bn_lif_forward(_neuron_id(spec, k), ctypes.byref(params), T, B, C, Lp, y.data_ptr(), bn_map[0].data_ptr(),
                                               bn_map[1].data_ptr(), v_keep.data_ptr(), None if packed else spikes.data_ptr(),
                                               spikes.data_ptr() if packed else None, v_last.data_ptr(), _stream(y))
        else:
            rc = L.load().sjhip_bn_plif_forward(ctypes.byref(params), T, B, C, Lp, y.data_ptr(), bn_map[0].data_ptr(),
                                                bn_map[1].data_ptr(), v_keep.data_ptr(), k_ptr,
                                                None if packed else spikes.data_ptr(), spikes.data_ptr() if packed else None,
                                                v_last.data_ptr(), _stream(y))
    L.check(rc, "bn_lif_forward")
    return spikes, v_last


def _bn_lif_backward(y: torch.Tensor, bn_map: torch.Tensor, gamma, v_init: torch.Tensor, spec, batch_stats: bool,
                     grad_spikes: Optional[torch.Tensor], grad_v_last: Optional[torch.Tensor], need_grad_v_init: bool,
                     want_amax: bool = False, k: Optional[torch.Tensor] = None):
    """Returns ``(dy [T, B, C, L], dgamma [C], dbeta [C], grad_v_init or None)``, and with ``want_amax`` a fifth element:
    ``amax(dy)``, found by the kernel that writes ``dy``, when the convolution GEMMs run on fp16 terms (else None).
    With ``k`` (parametric LIF) one more element follows: ``dL/dk``, one fp32 element."""
    T, B, C, Lp = y.shape
    lib = L.load()
    if grad_spikes is None:
        grad_spikes = torch.zeros_like(y)
    grad_spikes = L.aligned16(grad_spikes.to(torch.float32))
    if grad_v_last is not None:
        grad_v_last = L.aligned16(grad_v_last.to(torch.float32))
    v_keep, broadcast = K._state_arg(v_init, True)
    params = _lif_params(spec, broadcast)
    g = torch.empty_like(y)
    partial = torch.empty((B * C, 2), dtype=torch.float32, device=y.device)
    grads = torch.empty((5, C), dtype=torch.float32, device=y.device)  # dgamma, dbeta, then the coefficients p, q, r
    grad_v_init = torch.empty((B, C, Lp), dtype=torch.float32, device=y.device) if need_grad_v_init else None
    with torch.cuda.device(y.device):
        stream = _stream(y)
        grad_k = None
        if k is None:
            L.check(lib.sjhip_bn_lif_backward(_neuron_id(spec, k), ctypes.byref(params), T, B, C, Lp, y.data_ptr(), bn_map[0].data_ptr(),
                                              bn_map[1].data_ptr(), v_keep.data_ptr(), grad_spikes.data_ptr(), L.ptr(grad_v_last),
                                              g.data_ptr(), L.ptr(grad_v_init), partial.data_ptr(), stream), "bn_lif_backward")
        else:
            k_keep, k_ptr = K._k_pointer(k, y)
            grad_k = torch.empty((1,), dtype=torch.float32, device=y.device)
            shares = torch.empty((lib.sjhip_bn_plif_backward_workspace_floats(B, C, Lp),), dtype=torch.float32, device=y.device)
            L.check(lib.sjhip_bn_plif_backward(ctypes.byref(params), T, B, C, Lp, y.data_ptr(), bn_map[0].data_ptr(),
                                               bn_map[1].data_ptr(), v_keep.data_ptr(), k_ptr, grad_spikes.data_ptr(),
                                               L.ptr(grad_v_last), g.data_ptr(), L.ptr(grad_v_init), partial.data_ptr(),
                                               grad_k.data_ptr(), shares.data_ptr(), stream), "bn_plif_backward")
        dy_amax = None
        if want_amax and _terms() & F16:  # (cleared by the launch that makes the coefficients, filled by the next one)
            dy_amax = torch.empty((amax_floats(T * B),), dtype=torch.float32, device=y.device)
        L.check(lib.sjhip_bn_backward_finalize(partial.data_ptr(), T, B, C, Lp, 1 if batch_stats else 0, L.ptr(gamma),
                                               bn_map[2].data_ptr(), bn_map[3].data_ptr(), grads[0].data_ptr(),
                                               grads[1].data_ptr(), grads[2].data_ptr(), L.ptr(dy_amax), stream),
                "bn_backward_finalize")
        if dy_amax is not None:
            L.check(lib.sjhip_bn_grad_input_amax(g.data_ptr(), y.data_ptr(), grads[2].data_ptr(), T * B, C, Lp, g.data_ptr(),
                                                 dy_amax.data_ptr(), stream), "bn_grad_input_amax")
        else:
            L.check(lib.sjhip_bn_grad_input(g.data_ptr(), y.data_ptr(), grads[2].data_ptr(), T * B, C, Lp, g.data_ptr(), stream),
                    "bn_grad_input")
    out = (g, grads[0], grads[1], grad_v_init, dy_amax) if want_amax else (g, grads[0], grads[1], grad_v_init)
    return out if k is None else (*out, grad_k)


# ------------------------------------------------------------------------------------------------
# autograd
# ------------------------------------------------------------------------------------------------
# bn: (running_mean | None, running_var | None, batch_stats, momentum, eps[, num_batches_tracked | None])
# lif spec: (tau, v_threshold, v_reset, flags, sg_id, sg_alpha); tau = 0: an IF neuron, or with k a parametric LIF
def _bn_config(bn):
    """The batch-norm tuple with its optional sixth element (the counter of batches, incremented by the launch that
    updates the running statistics)."""
    return tuple(bn) if len(bn) == 6 else (*bn, None)


def _conv_forward(x_seq, weight, x_exact, stats: bool):
    """``(y [T, B, Cout, L], partial batch-norm sums of y or None, amax(x_seq) or an empty tensor)``: the last is what the
    fp16 split of a real-valued input was scaled by, which the weight gradient needs again."""
    T, B, Cin, Lp = x_seq.shape
    Cout = weight.shape[0]
    terms = _terms()
    x3 = x_seq.reshape(T * B, Cin, Lp)
    if terms & F16 and not x_exact:  # the split of the weights clears the buffer that the pass over x then fills
        x_amax = torch.empty((amax_floats(T * B),), dtype=torch.float32, device=x_seq.device)
        planes = split_weight(weight, False, terms, x_amax)
        amax(x3, x_amax)
    else:
        x_amax = x_seq.new_empty((0,))
        planes = split_weight(weight, False, terms)
    out = pw_gemm(planes, terms, Cout, Cin, x3, _exact(terms) if x_exact else terms, stats, x_amax if x_amax.numel() else None)
    if stats:
        return out[0].view(T, B, Cout, Lp), out[1], x_amax
    return out.view(T, B, Cout, Lp), None, x_amax


def _conv_backward(dy, x_seq, weight, x_exact, need_dx, need_dw, dy_amax=None, x_amax=None):
    T, B, Cin, Lp = x_seq.shape
    Cout = weight.shape[0]
    terms = _terms()
    dy3 = dy.view(T * B, Cout, Lp)
    if dy_amax is None and terms & F16 and (need_dw or need_dx):
        dy_amax = amax(dy3)  # one pass for both uses of dy
    if x_amax is not None and x_amax.numel() == 0:
        x_amax = None  # the forward ran with an exact input or on bf16 terms (pw_grad_weight finds it if it is needed now)
    x3 = x_seq.reshape(T * B, Cin, Lp)
    x_terms = _exact(terms) if x_exact else terms
    dw = dx = None
    if (need_dw and need_dx and getattr(configure, "hip_conv_overlap_gradients", False)
            and not torch.cuda.is_current_stream_capturing()):  # (a recorded graph keeps the step on the stream it records)
        # The two gradients only share their inputs: the weight gradient runs on a second stream, so that the blocks of
        # one kernel fill the compute units that the last, partly filled round of the other leaves idle.
        main = torch.cuda.current_stream(dy.device)
        side = _side_stream(dy.device)
        side.wait_stream(main)
        with torch.cuda.stream(side):
            dw = pw_grad_weight(dy3, terms, x3, x_terms, dy_amax, x_amax)
        dx = pw_gemm(split_weight(weight, True, terms), terms, Cin, Cout, dy3, terms, False, dy_amax).view(T, B, Cin, Lp)
        main.wait_stream(side)
        dw.record_stream(main)
        return dx, dw
    if need_dw:
        dw = pw_grad_weight(dy3, terms, x3, x_terms, dy_amax, x_amax)
    if need_dx:
        dx = pw_gemm(split_weight(weight, True, terms), terms, Cin, Cout, dy3, terms, False, dy_amax).view(T, B, Cin, Lp)
    return dx, dw


_SIDE_STREAMS: dict = {}


def _side_stream(device: torch.device) -> "torch.cuda.Stream":
    """One more stream per device (default priority), made on first use."""
    key = torch.device(device).index
    if key is None:
        key = torch.cuda.current_device()
    stream = _SIDE_STREAMS.get(key)
    if stream is None:
        stream = _SIDE_STREAMS[key] = torch.cuda.Stream(device=key)
    return stream


def _conv_chain_backward(x_seq, weight, gamma, v_init, y, bn_map, bits, x_amax, spec, batch_stats: bool, x_exact: bool, ssa,
                         grad_out, grad_v_last, need_dx: bool, need_dw: bool, need_gvi: bool, k=None):
    """Backward of convolution -> batch norm -> LIF (-> contraction on the bit-packed spikes when ``ssa = (heads,
    channels per head, scale)``): ``(dx, dw, dgamma, dbeta, grad_v_init)``, ``None`` where not needed; with ``k``
    (parametric LIF) a sixth element, ``dL/dk``."""
    grad_spikes = grad_out
    if ssa is not None and grad_out is not None:
        from . import attention_kernel as A

        heads, cph, scale = ssa
        T, B, _, Lp = x_seq.shape
        grad_spikes = A._ssa_packed(bits, grad_out, torch.float32, T * B, heads, cph, Lp, scale).view(y.shape)
    dy, dgamma, dbeta, gvi, dy_amax, *grad_k = _bn_lif_backward(y, bn_map, gamma, v_init, spec, batch_stats, grad_spikes,
                                                                 grad_v_last, need_gvi, True, k)
    dx, dw = _conv_backward(dy, x_seq, weight, x_exact, need_dx, need_dw, dy_amax, x_amax)
    return (dx, dw, dgamma, dbeta, gvi, *grad_k)


def _lif_conv_chain_backward(pre_seq, pre_v_init, weight, gamma, v_init, y, bn_map, bits, pre_spec, spec, batch_stats: bool,
                             grad_spikes, grad_v_last, grad_pre_v_last, need_gx: bool, need_gpv: bool, need_dw: bool,
                             need_gvi: bool, k=None):
    """Backward of LIF -> convolution -> batch norm -> LIF with the first neuron's spikes as bits:
    ``(grad of the first neuron's input, of its state, dw, dgamma, dbeta, grad_v_init)``; with ``k`` (the second neuron
    is a parametric LIF) a seventh element, ``dL/dk``."""
    T, B, Cin, Lp = pre_seq.shape
    Cout = weight.shape[0]
    terms = _terms()
    dy, dgamma, dbeta, gvi, dy_amax, *grad_k = _bn_lif_backward(y, bn_map, gamma, v_init, spec, batch_stats, grad_spikes,
                                                                 grad_v_last, need_gvi, True, k)
    dy3 = dy.view(T * B, Cout, Lp)
    if dy_amax is None:
        dy_amax = amax(dy3)
    dw = pw_grad_weight_bits(dy3, bits, Cin, dy_amax) if need_dw else None
    gx = gpv = None
    if need_gx or need_gpv:
        grad_pre_spikes = pw_gemm(split_weight(weight, True, terms), terms, Cin, Cout, dy3, terms, False, dy_amax)
        tau, v_th, v_reset, flags, sg_id, sg_alpha = pre_spec
        glast = grad_pre_v_last.flatten() if grad_pre_v_last is not None else None
        gx, gpv, _ = K._run_backward(L.NEURON_LIF, grad_pre_spikes.view(T, -1), None, glast, None, pre_seq.view(T, -1),
                                     pre_v_init.flatten(), None, tau, v_th, v_reset, flags, sg_id, sg_alpha, need_gpv)
        gx = gx.view(pre_seq.shape) if need_gx else None
        gpv = gpv.view(B, Cin, Lp) if need_gpv else None
    return (gx, gpv, dw, dgamma, dbeta, gvi, *grad_k)


class _BnLif(torch.autograd.Function):
    @staticmethod
    def forward(y, gamma, beta, v_init, bn, spec, k=None):
        running_mean, running_var, batch_stats, momentum, eps, tracked = _bn_config(bn)
        y = L.aligned16(y)
        bn_map = _bn_map(y.flatten(0, 1), gamma, beta, running_mean, running_var, batch_stats, momentum, eps, None, tracked)
        spikes, v_last = _bn_lif_forward(y, bn_map, v_init, spec, False, k)
        return spikes, v_last, bn_map

    @staticmethod
    def setup_context(ctx, inputs, output):
        y, gamma, beta, v_init, bn, spec, k = inputs
        ctx.spec, ctx.batch_stats = spec, bn[2]
        ctx.save_for_backward(L.aligned16(y), gamma, v_init, output[2], k)
        ctx.mark_non_differentiable(output[2])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_spikes, grad_v_last, _):
        y, gamma, v_init, bn_map, k = ctx.saved_tensors
        need = ctx.needs_input_grad
        dy, dgamma, dbeta, gvi, *grad_k = _bn_lif_backward(y, bn_map, gamma, v_init, ctx.spec, ctx.batch_stats, grad_spikes,
                                                           grad_v_last, bool(need[3]), False, k)
        return (dy if need[0] else None, dgamma if need[1] else None, dbeta if need[2] else None, gvi, None, None,
                grad_k[0] if grad_k and need[6] else None)


class _ConvBnLif(torch.autograd.Function):
    @staticmethod
    def forward(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, k=None):
        running_mean, running_var, batch_stats, momentum, eps, tracked = _bn_config(bn)
        x_seq = L.aligned16(x_seq)
        y, partial, x_amax = _conv_forward(x_seq, weight, x_exact, batch_stats)
        bn_map = _bn_map(y.flatten(0, 1), gamma, beta, running_mean, running_var, batch_stats, momentum, eps, partial, tracked)
        spikes, v_last = _bn_lif_forward(y, bn_map, v_init, spec, False, k)
        return spikes, v_last, y, bn_map, x_amax

    @staticmethod
    def setup_context(ctx, inputs, output):
        x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, k = inputs
        ctx.spec, ctx.batch_stats, ctx.x_exact = spec, bn[2], x_exact
        ctx.save_for_backward(L.aligned16(x_seq), weight, gamma, v_init, output[2], output[3], output[4], k)
        ctx.mark_non_differentiable(output[2], output[3], output[4])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_spikes, grad_v_last, _y, _map, _amax):
        x_seq, weight, gamma, v_init, y, bn_map, x_amax, k = ctx.saved_tensors
        need = ctx.needs_input_grad
        dx, dw, dgamma, dbeta, gvi, *grad_k = _conv_chain_backward(x_seq, weight, gamma, v_init, y, bn_map, None, x_amax,
                                                                   ctx.spec, ctx.batch_stats, ctx.x_exact, None, grad_spikes,
                                                                   grad_v_last, bool(need[0]), bool(need[1]), bool(need[4]), k)
        return (dx, dw, dgamma if need[2] else None, dbeta if need[3] else None, gvi, None, None, None,
                grad_k[0] if grad_k and need[8] else None)


class _ConvBnLifSsa(torch.autograd.Function):
    """The qkv half of the spiking self-attention: convolution, batch norm, LIF with bit-packed spike output, and the
    contraction ``scale (V K^T) Q`` reading those bits.  Saves the input, the convolution output and the bits."""

    @staticmethod
    def forward(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, ssa, k=None):
        from . import attention_kernel as A

        running_mean, running_var, batch_stats, momentum, eps, tracked = _bn_config(bn)
        heads, cph, scale = ssa
        x_seq = L.aligned16(x_seq)
        T, B, _, Lp = x_seq.shape
        y, partial, x_amax = _conv_forward(x_seq, weight, x_exact, batch_stats)
        bn_map = _bn_map(y.flatten(0, 1), gamma, beta, running_mean, running_var, batch_stats, momentum, eps, partial, tracked)
        bits, v_last = _bn_lif_forward(y, bn_map, v_init, spec, True, k)
        out = A._ssa_packed(bits, None, torch.float32, T * B, heads, cph, Lp, scale)
        return out, v_last, y, bn_map, bits, x_amax

    @staticmethod
    def setup_context(ctx, inputs, output):
        x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, ssa, k = inputs
        ctx.spec, ctx.batch_stats, ctx.x_exact, ctx.ssa = spec, bn[2], x_exact, ssa
        ctx.save_for_backward(L.aligned16(x_seq), weight, gamma, v_init, output[2], output[3], output[4], output[5], k)
        ctx.mark_non_differentiable(output[2], output[3], output[4], output[5])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_out, grad_v_last, _y, _map, _bits, _amax):
        from . import attention_kernel as A

        x_seq, weight, gamma, v_init, y, bn_map, bits, x_amax, k = ctx.saved_tensors
        need = ctx.needs_input_grad
        dx, dw, dgamma, dbeta, gvi, *grad_k = _conv_chain_backward(x_seq, weight, gamma, v_init, y, bn_map, bits, x_amax,
                                                                   ctx.spec, ctx.batch_stats, ctx.x_exact, ctx.ssa, grad_out,
                                                                   grad_v_last, bool(need[0]), bool(need[1]), bool(need[4]), k)
        return (dx, dw, dgamma if need[2] else None, dbeta if need[3] else None, gvi, None, None, None, None,
                grad_k[0] if grad_k and need[9] else None)


class _ConvBnLifSsaLif(torch.autograd.Function):
    """``_ConvBnLifSsa`` followed by the attention's own LIF, whose input ``scale (V K^T) Q`` never leaves the kernel
    that computes it.  Saves the input, the convolution output, the bits and, when a gradient is wanted, the attention
    neuron's ``h_seq``."""

    @staticmethod
    def forward(x_seq, weight, gamma, beta, v_init, attn_v_init, bn, spec, x_exact, ssa, attn_spec, save_h):
        from . import attention_kernel as A

        running_mean, running_var, batch_stats, momentum, eps, tracked = _bn_config(bn)
        heads, cph, scale = ssa
        x_seq = L.aligned16(x_seq)
        T, B, _, Lp = x_seq.shape
        y, partial, x_amax = _conv_forward(x_seq, weight, x_exact, batch_stats)
        bn_map = _bn_map(y.flatten(0, 1), gamma, beta, running_mean, running_var, batch_stats, momentum, eps, partial, tracked)
        bits, v_last = _bn_lif_forward(y, bn_map, v_init, spec, True)
        v_keep, broadcast = K._state_arg(attn_v_init, True)
        spikes, h_seq, attn_v_last = A._ssa_lif_forward(bits, v_keep, _lif_params(attn_spec, broadcast), T, B, heads, cph,
                                                        Lp, scale, save_h)
        if h_seq is None:
            h_seq = spikes.new_empty((0,))
        return spikes, v_last, attn_v_last, y, bn_map, bits, h_seq, x_amax

    @staticmethod
    def setup_context(ctx, inputs, output):
        x_seq, weight, gamma, beta, v_init, attn_v_init, bn, spec, x_exact, ssa, attn_spec, save_h = inputs
        ctx.spec, ctx.batch_stats, ctx.x_exact, ctx.ssa, ctx.attn_spec = spec, bn[2], x_exact, ssa, attn_spec
        ctx.save_for_backward(L.aligned16(x_seq), weight, gamma, v_init, output[3], output[4], output[5], output[6], output[7])
        ctx.mark_non_differentiable(output[3], output[4], output[5], output[6], output[7])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_attn_spikes, grad_v_last, grad_attn_v_last, _y, _map, _bits, _h, _amax):
        from . import attention_kernel as A

        x_seq, weight, gamma, v_init, y, bn_map, bits, h_seq, x_amax = ctx.saved_tensors
        if h_seq.numel() == 0:
            raise RuntimeError("the fused attention block was run without saving h_seq and cannot be differentiated")
        heads, cph, scale = ctx.ssa
        T, B, _, Lp = x_seq.shape
        need = ctx.needs_input_grad
        grad_spikes = None
        if grad_attn_spikes is not None or grad_attn_v_last is not None:
            grad_qkv, _ = A._ssa_lif_backward(bits, h_seq, grad_attn_spikes, grad_attn_v_last, _lif_params(ctx.attn_spec), T, B,
                                              heads, cph, Lp, scale, False)
            grad_spikes = grad_qkv.view(y.shape)
        dy, dgamma, dbeta, gvi, dy_amax = _bn_lif_backward(y, bn_map, gamma, v_init, ctx.spec, ctx.batch_stats, grad_spikes,
                                                            grad_v_last, bool(need[4]), True)
        dx, dw = _conv_backward(dy, x_seq, weight, ctx.x_exact, bool(need[0]), bool(need[1]), dy_amax, x_amax)
        return (dx, dw, dgamma if need[2] else None, dbeta if need[3] else None, gvi, None, None, None, None, None, None, None)


class _LifConvBnLif(torch.autograd.Function):
    """A multi-step LIF whose spikes feed a kernel-size-1 convolution, batch norm and a second LIF, with those spikes
    existing only bit-packed: the first neuron writes bits (``sjhip_neuron_forward_packed``), the convolution and its
    weight gradient read bits, and the first neuron's backward replays its forward from its input.  This is the
    ``attn_lif -> proj_conv -> proj_bn -> proj_lif`` tail of the spiking self-attention (reference
    layer/attention.py:376-384).  Saves the first neuron's input, the bits (1/32 of the fp32 spike tensor), the
    convolution output and the batch-norm map."""

    @staticmethod
    def forward(pre_seq, pre_v_init, weight, gamma, beta, v_init, bn, pre_spec, spec, k=None):
        running_mean, running_var, batch_stats, momentum, eps, tracked = _bn_config(bn)
        pre_seq = L.aligned16(pre_seq)
        T, B, Cin, Lp = pre_seq.shape
        Cout = weight.shape[0]
        tau, v_th, v_reset, flags, _, _ = pre_spec
        bits, _, pre_v_last = K._run_forward_packed(L.NEURON_LIF, pre_seq.view(T, -1), pre_v_init.flatten(), None, tau, v_th,
                                                    v_reset, flags, False)
        terms = _terms()
        planes = split_weight(weight, False, terms)
        out = pw_gemm_bits(planes, Cout, Cin, bits, T * B, Lp, batch_stats)
        y, partial = (out[0], out[1]) if batch_stats else (out, None)
        y = y.view(T, B, Cout, Lp)
        bn_map = _bn_map(y.flatten(0, 1), gamma, beta, running_mean, running_var, batch_stats, momentum, eps, partial, tracked)
        spikes, v_last = _bn_lif_forward(y, bn_map, v_init, spec, False, k)
        return spikes, v_last, pre_v_last.view(B, Cin, Lp), y, bn_map, bits

    @staticmethod
    def setup_context(ctx, inputs, output):
        pre_seq, pre_v_init, weight, gamma, beta, v_init, bn, pre_spec, spec, k = inputs
        ctx.pre_spec, ctx.spec, ctx.batch_stats = pre_spec, spec, _bn_config(bn)[2]
        ctx.save_for_backward(L.aligned16(pre_seq), pre_v_init, weight, gamma, v_init, output[3], output[4], output[5], k)
        ctx.mark_non_differentiable(output[3], output[4], output[5])
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, grad_spikes, grad_v_last, grad_pre_v_last, _y, _map, _bits):
        pre_seq, pre_v_init, weight, gamma, v_init, y, bn_map, bits, k = ctx.saved_tensors
        need = ctx.needs_input_grad
        gx, gpv, dw, dgamma, dbeta, gvi, *grad_k = _lif_conv_chain_backward(
            pre_seq, pre_v_init, weight, gamma, v_init, y, bn_map, bits, ctx.pre_spec, ctx.spec, ctx.batch_stats, grad_spikes,
            grad_v_last, grad_pre_v_last, bool(need[0]), bool(need[1]), bool(need[2]), bool(need[5]), k)
        return (gx, gpv, dw, dgamma if need[3] else None, dbeta if need[4] else None, gvi, None, None, None,
                grad_k[0] if grad_k and need[9] else None)


def lif_conv_bn_lif(pre_seq: torch.Tensor, pre_v_init: torch.Tensor, weight: torch.Tensor, gamma, beta, v_init: torch.Tensor,
                    bn, pre_spec, spec, k: Optional[torch.Tensor] = None):
    """``pre_seq [T, B, Cin, L]`` is the input of a LIF (``pre_spec``, state ``pre_v_init [B, Cin, L]``) whose spikes go
    through ``weight [Cout, Cin]``, batch norm and a second LIF (``spec``, ``v_init [B, Cout, L]``).  Returns
    ``(spikes [T, B, Cout, L], v_last, v_last of the first neuron)``.  The caller has checked ``lif_conv_bn_lif_supported``."""
    if torch.compiler.is_compiling():
        from . import fused_ops as O

        return O.lif_conv_bn_lif(pre_seq, pre_v_init, weight, gamma, beta, v_init, bn, pre_spec, spec, k)
    out = _LifConvBnLif.apply(pre_seq, pre_v_init, weight, gamma, beta, v_init, bn, pre_spec, spec, k)
    return out[0], out[1], out[2]


def lif_conv_bn_lif_supported(pre_seq: torch.Tensor, need_grad: bool) -> bool:
    """What ``supported`` asks, the fp16 split of the GEMM operands (the kernels that read bits belong to it) and a
    spike tensor whose samples start on a byte."""
    if not supported(pre_seq, need_grad) or not (_terms() & F16):
        return False
    T, B, Cin, Lp = pre_seq.shape
    return (Cin * Lp) % 8 == 0


def bn_lif(y_seq: torch.Tensor, gamma, beta, v_init: torch.Tensor, bn, spec, k: Optional[torch.Tensor] = None):
    """``y_seq [T, B, C, L]`` (a convolution output) -> ``(spikes, v_last)``.  ``k``: ``sigmoid(w)`` of a parametric LIF
    (one element on the device; its gradient comes back through autograd), in which case ``spec[0]`` is unused."""
    if torch.compiler.is_compiling():
        from . import fused_ops as O

        return O.bn_lif(y_seq, gamma, beta, v_init, bn, spec, k)
    spikes, v_last, _ = _BnLif.apply(y_seq, gamma, beta, v_init, bn, spec, k)
    return spikes, v_last


def conv_bn_lif(x_seq: torch.Tensor, weight: torch.Tensor, gamma, beta, v_init: torch.Tensor, bn, spec, x_exact: bool,
                k: Optional[torch.Tensor] = None):
    """``x_seq [T, B, Cin, L]``, ``weight [Cout, Cin]`` -> ``(spikes [T, B, Cout, L], v_last [B, Cout, L])``.
    ``x_exact``: every element of ``x_seq`` is exactly representable in bf16 (spikes, small integers)."""
    if torch.compiler.is_compiling():
        from . import fused_ops as O

        return O.conv_bn_lif(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, None, k)
    spikes, v_last, _, _, _ = _ConvBnLif.apply(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, k)
    return spikes, v_last


def conv_bn_lif_ssa(x_seq: torch.Tensor, weight: torch.Tensor, gamma, beta, v_init: torch.Tensor, bn, spec, x_exact: bool,
                    heads: int, channels_per_head: int, scale: float, k: Optional[torch.Tensor] = None):
    """The same block with ``Cout = 3 * heads * channels_per_head`` followed by the contraction; returns
    ``(out [T * B, heads, channels_per_head, L], v_last)``."""
    if torch.compiler.is_compiling():
        from . import fused_ops as O

        return O.conv_bn_lif(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact, (heads, channels_per_head, scale), k)
    out, v_last, _, _, _, _ = _ConvBnLifSsa.apply(x_seq, weight, gamma, beta, v_init, bn, spec, x_exact,
                                               (heads, channels_per_head, scale), k)
    return out, v_last


def conv_bn_lif_ssa_lif(x_seq: torch.Tensor, weight: torch.Tensor, gamma, beta, v_init: torch.Tensor, attn_v_init: torch.Tensor,
                        bn, spec, x_exact: bool, heads: int, channels_per_head: int, scale: float, attn_spec, save_h: bool):
    """``conv_bn_lif_ssa`` followed by the LIF of ``attn_spec`` on the contraction's output; returns
    ``(spikes [T, B, heads, channels_per_head, L], v_last of the first neuron, v_last of the attention neuron)``."""
    out = _ConvBnLifSsaLif.apply(x_seq, weight, gamma, beta, v_init, attn_v_init, bn, spec, x_exact,
                                 (heads, channels_per_head, scale), attn_spec, save_h)
    return out[0], out[1], out[2]
