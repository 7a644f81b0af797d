"""torch-ops restatement of the reference's ST-BIF step (CPU).  Test infrastructure only.

Paths relative to ``spikingjelly/activation_based``.  ``step`` follows ``functional/neuron.py:3234-3247`` line by
line (the torch backend, every op in the tensor's dtype); ``multi_step_fp32_state`` follows the Triton kernel
``triton_kernel/neuron_kernel/stbif.py:94-137`` with the host code at ``:360-362`` (scalars rounded to the storage
dtype, fp32 arithmetic and state, stored values rounded).
"""

from __future__ import annotations

import torch


def step(x, q, acc_q, q_threshold, pos_max, neg_min):
    q_threshold = q_threshold.to(x)  # :3234-3236
    pos_max = pos_max.to(x)
    neg_min = neg_min.to(x)
    normalized = x / q_threshold  # :3237
    q_next = q + normalized.detach()  # :3238
    acc_q_next = torch.round(acc_q)  # :3239
    spike_position = (q_next - 1 >= 0) & (acc_q_next < pos_max)  # :3240
    neg_spike_position = (q_next < 0) & (acc_q_next > neg_min)  # :3241
    cur_output_next = spike_position.to(x.dtype) - neg_spike_position.to(x.dtype)  # :3242
    acc_q_next = acc_q_next + cur_output_next  # :3243
    q_next = torch.where(spike_position, q_next - 1, q_next)  # :3244
    q_next = torch.where(neg_spike_position, q_next + 1, q_next)  # :3245
    out = cur_output_next * q_threshold  # :3246
    return out, q_next, acc_q_next, cur_output_next


def multi_step(x_seq, q, acc_q, q_threshold, pos_max, neg_min):
    """Step loop of ``neuron/spikezip.py:331-345``: (out_seq, q, acc_q, cur_output, is_work)."""
    out_seq = torch.empty_like(x_seq)
    cur = torch.zeros_like(x_seq[0])
    for t in range(x_seq.shape[0]):
        out_seq[t], q, acc_q, cur = step(x_seq[t], q, acc_q, q_threshold, pos_max, neg_min)
    return out_seq, q, acc_q, cur, bool((x_seq != 0).any() | (out_seq != 0).any())


def multi_step_fp32_state(x_seq, q, acc_q, q_threshold, pos_max, neg_min):
    """The Triton kernel's arithmetic: returns tensors of ``x_seq``'s dtype."""
    dtype = x_seq.dtype
    s, hi, lo = (float(v.to(dtype)) for v in (q_threshold, pos_max, neg_min))  # stbif.py:360-362
    x32, q, acc_q = x_seq.float(), q.float(), acc_q.float()
    out_seq = torch.empty_like(x32)
    cur = torch.zeros_like(q)
    for t in range(x32.shape[0]):
        normalized = x32[t] / s
        q = q + normalized
        acc_q = torch.round(acc_q)
        pos = (q >= 1.0) & (acc_q < hi)
        neg = (q < 0.0) & (acc_q > lo)
        cur = pos.float() - neg.float()
        acc_q = acc_q + cur
        q = q - pos.float() + neg.float()
        out_seq[t] = cur * s
    return out_seq.to(dtype), q.to(dtype), acc_q.to(dtype), cur.to(dtype)
