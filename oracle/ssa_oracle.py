"""CPU restatement of the spiking self-attention contraction.  Test infrastructure only.

Follows ``SpikingSelfAttention._ssa_kernel_torch`` of the reference
(``spikingjelly/activation_based/layer/attention.py:346-353``):

    qt, kt, vt = qkv.flatten(2, 3).chunk(3, dim=2)      # each [T, N, heads, Cph, L]
    x_seq = vt @ kt.transpose(-2, -1)                   # [.., Cph, Cph]
    x_seq = (x_seq @ qt) * scale                        # [.., Cph, L]

here on ``qkv`` of shape ``[S, 3, H, Cph, L]`` (T and N already folded into S).  ``ssa_exact`` does the two
products in int64 (the inputs are binary spikes, so this is the exact value any fp32-accumulating
implementation must return); ``ssa`` runs the same ops in the tensor's own dtype and is differentiable.
"""

from __future__ import annotations

import torch


def ssa(qkv: torch.Tensor, scale: float) -> torch.Tensor:
    qt, kt, vt = qkv[:, 0], qkv[:, 1], qkv[:, 2]
    x = vt @ kt.transpose(-2, -1)
    return (x @ qt) * scale


def ssa_exact(qkv: torch.Tensor, scale: float) -> torch.Tensor:
    """float64 tensor holding scale * (V K^T) Q computed in integers."""
    q, k, v = (qkv[:, i].to(torch.int64) for i in range(3))
    s = v @ k.transpose(-2, -1)
    return (s @ q).to(torch.float64) * scale
