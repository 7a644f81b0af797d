"""CPU restatement of ``Conv1d(k=1, bias=False) -> BatchNorm1d -> LIFNode`` and of the whole spiking self-attention
block.  Test infrastructure only: nothing under ``spikingjelly_amd/`` imports this file.

Follows the reference's ``SpikingSelfAttention`` (``layer/attention.py:310-329`` construction, ``:346-353`` contraction,
``:355-384`` forward): ``SeqToANNContainer`` folds time into the batch (``layer/container.py:66``), the convolution and
the batch norm are torch's own modules, the neurons are ``LIFNode(tau=2, detach_reset=True)`` with the default
``Sigmoid(4)`` surrogate (``attn_lif`` with ``v_threshold=0.5``).  Everything is written with plain tensor algebra
(``einsum``, mean / variance by their definitions) instead of ``F.conv1d`` / ``F.batch_norm`` so that the test that
compares the two pins this file against torch's operators, and runs in whatever dtype the inputs have (float64 for
the accuracy reference).
"""

from __future__ import annotations

from typing import Optional

import torch

from . import neuron_oracle as no


def pointwise_conv(x_seq: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``x_seq [T, B, Cin, L]``, ``weight [Cout, Cin]`` -> ``[T, B, Cout, L]``: ``nn.Conv1d(kernel_size=1, bias=False)``
    applied to every time step."""
    return torch.einsum("oc,tbcl->tbol", weight, x_seq)


def batch_norm(y_seq: torch.Tensor, gamma: Optional[torch.Tensor], beta: Optional[torch.Tensor],
               running_mean: Optional[torch.Tensor], running_var: Optional[torch.Tensor], training: bool,
               momentum: float = 0.1, eps: float = 1e-5):
    """``nn.BatchNorm1d`` over the channel axis of ``[T, B, C, L]`` (time folded into the batch).  Returns
    ``(z, new_running_mean, new_running_var)``; the running statistics are returned, not modified."""
    C = y_seq.shape[2]
    if training or running_mean is None:
        flat = y_seq.transpose(0, 2).reshape(C, -1)  # [C, T*B*L]
        n = flat.shape[1]
        mean = flat.mean(dim=1)
        var = ((flat - mean[:, None]) ** 2).mean(dim=1)  # biased, used for normalising
        new_mean, new_var = running_mean, running_var
        if running_mean is not None and training:
            new_mean = (1 - momentum) * running_mean + momentum * mean
            new_var = (1 - momentum) * running_var + momentum * var * n / max(n - 1, 1)
    else:
        mean, var = running_mean, running_var
        new_mean, new_var = running_mean, running_var
    z = (y_seq - mean[None, None, :, None]) / torch.sqrt(var[None, None, :, None] + eps)
    if gamma is not None:
        z = z * gamma[None, None, :, None]
    if beta is not None:
        z = z + beta[None, None, :, None]
    return z, new_mean, new_var


def lif(z_seq: torch.Tensor, v_init: torch.Tensor, tau: float = 2.0, v_threshold: float = 1.0,
        v_reset: Optional[float] = 0.0, detach_reset: bool = True, sg_name: str = "sigmoid", sg_alpha: float = 4.0,
        decay_input: bool = True):
    """Multi-step LIF on ``[T, ...]``; returns ``(spike_seq, v_seq, h_seq)`` of the same shape."""
    shape = z_seq.shape
    s, v, h = no.multi_step("lif", z_seq.flatten(1), v_init.flatten(), tau, decay_input, v_threshold, v_reset,
                            no.surrogate(sg_name, sg_alpha), detach_reset)
    return s.reshape(shape), v.reshape(shape), h.reshape(shape)


def conv_bn_lif(x_seq, weight, gamma, beta, running_mean, running_var, training, v_init, momentum=0.1, eps=1e-5, **lif_kw):
    """Returns dict(y, z, spike_seq, v_seq, h_seq, running_mean, running_var)."""
    y = pointwise_conv(x_seq, weight)
    z, rm, rv = batch_norm(y, gamma, beta, running_mean, running_var, training, momentum, eps)
    s, v, h = lif(z, v_init, **lif_kw)
    return dict(y=y, z=z, spike_seq=s, v_seq=v, h_seq=h, running_mean=rm, running_var=rv)


def ssa_contraction(qkv_spikes: torch.Tensor, heads: int, scale: float) -> torch.Tensor:
    """``[T, B, 3*C, L]`` spikes -> ``[T, B, heads, C/heads, L]``: ``scale * (V K^T) Q`` per head
    (``layer/attention.py:346-353``)."""
    T, B, C3, L = qkv_spikes.shape
    qkv = qkv_spikes.reshape(T, B, 3, heads, C3 // 3 // heads, L)
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    return ((v @ k.transpose(-2, -1)) @ q) * scale


def attention_block(x_seq, params, heads: int, training: bool, momentum=0.1, eps=1e-5, scale: float = 0.125):
    """The whole ``SpikingSelfAttention.forward``.  ``params``: dict with ``qkv_weight [3C, C]``, ``qkv_gamma``, ``qkv_beta``,
    ``qkv_running_mean``, ``qkv_running_var``, and the same five with prefix ``proj_``.  All three neurons start from
    rest.  Returns dict with every intermediate (``qkv_h``, ``attn_h``, ``proj_h`` are the membrane potentials before
    firing, for margin checks)."""
    T, B, C, L = x_seq.shape
    zeros = lambda ch: torch.zeros((B, ch, L), dtype=x_seq.dtype)
    a = conv_bn_lif(x_seq, params["qkv_weight"], params["qkv_gamma"], params["qkv_beta"], params["qkv_running_mean"],
                    params["qkv_running_var"], training, zeros(3 * C), momentum, eps)
    out = ssa_contraction(a["spike_seq"], heads, scale)
    s_attn, _, h_attn = lif(out.reshape(T, B, C, L), zeros(C), v_threshold=0.5)
    b = conv_bn_lif(s_attn, params["proj_weight"], params["proj_gamma"], params["proj_beta"], params["proj_running_mean"],
                    params["proj_running_var"], training, zeros(C), momentum, eps)
    return dict(out=b["spike_seq"], qkv_h=a["h_seq"], attn_h=h_attn, proj_h=b["h_seq"], qkv_spikes=a["spike_seq"],
                attn_spikes=s_attn, ssa=out, qkv_y=a["y"], proj_y=b["y"],
                qkv_running=(a["running_mean"], a["running_var"]), proj_running=(b["running_mean"], b["running_var"]))
