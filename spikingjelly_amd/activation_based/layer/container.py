"""``SeqToANNContainer``: run stateless layers on a ``[T, N, ...]`` sequence by folding time into the
batch (reference ``layer/container.py:66`` and ``functional/forward.py:316-321``)."""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import base


class SeqToANNContainer(nn.Sequential, base.MultiStepModule):
    def forward(self, x_seq: torch.Tensor):
        y = super().forward(x_seq.flatten(0, 1))
        return y.view(x_seq.shape[0], x_seq.shape[1], *y.shape[1:])
