"""Signed ternary BIF neuron of SpikeZIP's QANN-to-SNN conversion (reference ``neuron/spikezip.py:14-228``)."""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import base, functional

__all__ = ["STBIFNeuron"]


def _scalar_tensor(value) -> torch.Tensor:
    return (value if torch.is_tensor(value) else torch.tensor(value)).detach().clone().float()


class STBIFNeuron(base.MemoryModule):
    """Executes a quantised activation (scale ``q_threshold``, ``level`` integer levels, symmetric or not) as a spike
    train: each step emits ``-q_threshold``, ``0`` or ``+q_threshold``, and the emitted total converges to the
    quantiser's output for the accumulated input.  States: the residual ``q`` (starts at 0.5, i.e. round to
    nearest), the released integer ``acc_q`` (kept within ``[neg_min, pos_max]``), the last ternary output
    ``cur_output`` and ``is_work`` (whether the last call saw any non-zero input or output).  Inference only.
    Backends: ``'torch'`` and ``'hip'`` in both step modes (the reference offers ``'torch'`` and ``'triton'``).
    """

    def __init__(self, q_threshold, level: int, sym: bool = False, pos_max=None, neg_min=None, step_mode: str = "s"):
        super().__init__()
        self.level = int(level)
        if isinstance(level, bool) or self.level < 2:
            raise ValueError("SpikeZIP quantizer level must be >= 2.")
        self.sym = bool(sym)
        if pos_max is None:
            pos_max = self.level // 2 - 1 if self.sym else self.level - 1
        if neg_min is None:
            neg_min = -self.level // 2 if self.sym else 0
        self.register_buffer("q_threshold", _scalar_tensor(q_threshold))
        self.register_buffer("pos_max", _scalar_tensor(pos_max))
        self.register_buffer("neg_min", _scalar_tensor(neg_min))
        self.step_mode = step_mode
        self.register_memory("q", None)
        self.register_memory("acc_q", None)
        self.register_memory("cur_output", None)
        self.register_memory("is_work", False)

    @classmethod
    def from_quantizer(cls, quantizer: nn.Module) -> "STBIFNeuron":
        """From a SpikeZIP quantiser module exposing ``s``, ``sym``, ``pos_max``, ``neg_min`` and optionally
        ``level`` (otherwise the number of integers between the bounds)."""
        pos_max, neg_min = quantizer.pos_max, quantizer.neg_min
        span = int(_scalar_tensor(pos_max).item()) - int(_scalar_tensor(neg_min).item()) + 1
        return cls(quantizer.s, level=int(getattr(quantizer, "level", span)), sym=bool(quantizer.sym),
                   pos_max=pos_max, neg_min=neg_min)

    @property
    def supported_backends(self):
        return ("torch", "hip")

    def _fresh(self, x: torch.Tensor, value: float) -> torch.Tensor:
        # the hip kernel reads a constant state from one element: no [N] tensor is filled or read
        if self.backend == "hip" and x.is_cuda and x.numel() > 1:
            return x.new_full((1,) * x.dim(), value).expand(x.shape)
        return torch.full_like(x, value)

    def materialize_states(self, inputs, states, step_mode: str):
        x = inputs[0] if step_mode == "s" else inputs[0][0]
        q, acc_q, cur_output, is_work = states
        if q is None or q.shape != x.shape:
            q, acc_q, cur_output = self._fresh(x, 0.5), self._fresh(x, 0.0), torch.zeros_like(x)
        else:
            q, acc_q, cur_output = q.to(x), acc_q.to(x), cur_output.to(x)
        return q, acc_q, cur_output, is_work

    def single_step_functional_forward(self, inputs, states, **kwargs):
        x = inputs[0]
        q, acc_q, cur_output, is_work = states
        if self.backend == "hip":
            out, q, acc_q, cur_output, work = functional.stbif_single_step_hip(x, q, acc_q, self.q_threshold,
                                                                               self.pos_max, self.neg_min)
            return (out,), (q, acc_q, cur_output, bool(work.item()))
        out, q, acc_q, cur_output = functional.stbif_step(x, q, acc_q, self.q_threshold, self.pos_max, self.neg_min)
        return (out,), (q, acc_q, cur_output, bool((x != 0).any() | (out != 0).any()))

    def multi_step_functional_forward(self, inputs, states, **kwargs):
        x_seq = inputs[0]
        q, acc_q, cur_output, is_work = states
        if self.backend == "hip":
            out_seq, q, acc_q, cur_output, work = functional.stbif_multi_step_hip(x_seq, q, acc_q, self.q_threshold,
                                                                                  self.pos_max, self.neg_min)
            return (out_seq,), (q, acc_q, cur_output, bool(work.item()))
        out_seq = torch.empty_like(x_seq)
        for t in range(x_seq.shape[0]):
            out_seq[t], q, acc_q, cur_output = functional.stbif_step(x_seq[t], q, acc_q, self.q_threshold,
                                                                     self.pos_max, self.neg_min)
        return (out_seq,), (q, acc_q, cur_output, bool((x_seq != 0).any() | (out_seq != 0).any()))

    @property
    def accumulated(self) -> torch.Tensor:
        """The value released so far, ``acc_q * q_threshold``."""
        if self.acc_q is None:
            raise RuntimeError("STBIFNeuron has no accumulated state before forward.")
        return self.acc_q * self.q_threshold.to(dtype=self.acc_q.dtype)
