"""Quantisers with straight-through gradients used by the neurons of this package.

Only what the integer-valued LIF needs: the multi-level spike count of the reference's
``spikingjelly/activation_based/quantize.py:580-616``.
"""

from __future__ import annotations

from typing import Optional

import torch

__all__ = ["multi_level_spike_count"]


class _MultiLevelSpikeCount(torch.autograd.Function):
    """Forward ``round(clamp(x, 0, D))`` (ties to even); backward passes the gradient where
    ``grad_min <= x <= grad_max`` and blocks it elsewhere."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, max_spike_count: int, grad_min: float, grad_max: float):
        ctx.save_for_backward(x)
        ctx.window = (grad_min, grad_max)
        return torch.round(torch.clamp(x, 0, max_spike_count))

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        (x,) = ctx.saved_tensors
        lo, hi = ctx.window
        inside = (x >= lo) & (x <= hi)
        return grad_output * inside.to(grad_output.dtype), None, None, None


def multi_level_spike_count(x: torch.Tensor, max_spike_count: int,
                            grad_window: Optional[tuple[float, float]] = None) -> torch.Tensor:
    """Integer count in ``{0, ..., max_spike_count}`` nearest to ``x``; the gradient window defaults to
    ``[0, max_spike_count]``."""
    max_spike_count = int(max_spike_count)
    lo, hi = (0.0, float(max_spike_count)) if grad_window is None else grad_window
    return _MultiLevelSpikeCount.apply(x, max_spike_count, lo, hi)
