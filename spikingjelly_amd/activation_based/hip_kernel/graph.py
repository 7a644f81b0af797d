"""HIP graph capture of a step that runs through the hip backend.

The operators of this backend launch on the current stream, never synchronise the host and allocate through torch only,
so a whole step (a multi-step forward + backward, or a Python loop of single steps with its backward) can be recorded
once and replayed; for small layers that removes the per-launch host cost, which is what bounds a loop of single steps.
The reference reaches for ``torch.compile`` here (``test_compile_compat.py:125-170``); on this hardware a recorded graph
does the same job without a tracing compiler.

Rules of a recorded step (torch's, restated): it must do the same work every time (no data-dependent Python control
flow, no host reads of device values), its inputs live in fixed buffers that :meth:`GraphedStep.__call__` fills, and its
results are fixed buffers too, overwritten by every replay.
"""

from __future__ import annotations

from typing import Callable, Iterable, Optional, Sequence

import torch

__all__ = ["GraphedStep"]


def _clear_grads(tensors: Iterable[torch.Tensor]) -> None:
    for t in tensors:
        t.grad = None


class GraphedStep:
    """``step(*inputs)`` recorded into one HIP graph.

    :param step: the work to record; called with the static inputs.  It may run a backward pass; gradients then land in
        the ``.grad`` of the static inputs and of ``parameters`` (written, not accumulated, by every replay, because
        those ``.grad`` are cleared before recording and so are allocated inside the graph).
    :param example_inputs: tensors on the GPU; clones of them become the static inputs (``requires_grad`` is kept).
    :param parameters: parameters whose ``.grad`` the step produces.
    :param warmup: eager runs on a side stream before recording, as torch's capture protocol asks (lazy initialisation
        of libraries and of autograd must not happen while recording).

    Calling the object copies new inputs into the static ones, replays and returns what ``step`` returned while being
    recorded (the same tensors every time).  ``static_inputs`` exposes the input buffers (for their ``.grad``).
    """

    def __init__(self, step: Callable, example_inputs: Sequence[torch.Tensor],
                 parameters: Optional[Iterable[torch.Tensor]] = None, warmup: int = 3):
        if not example_inputs or not all(torch.is_tensor(t) and t.is_cuda for t in example_inputs):
            raise ValueError("GraphedStep records GPU work: every example input must be a tensor on the GPU")
        self.parameters = list(parameters) if parameters is not None else []
        self.static_inputs = [t.detach().clone().requires_grad_(t.requires_grad) for t in example_inputs]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):
                step(*self.static_inputs)
                _clear_grads(self.static_inputs)
                _clear_grads(self.parameters)
        torch.cuda.current_stream().wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.static_outputs = step(*self.static_inputs)

    def __call__(self, *inputs: torch.Tensor):
        if len(inputs) != len(self.static_inputs):
            raise ValueError(f"recorded with {len(self.static_inputs)} inputs, called with {len(inputs)}")
        with torch.no_grad():
            for static, new in zip(self.static_inputs, inputs):
                if static.shape != new.shape or static.dtype != new.dtype:
                    raise ValueError(f"recorded with {tuple(static.shape)} {static.dtype}, "
                                     f"called with {tuple(new.shape)} {new.dtype}")
                static.copy_(new)
        self.graph.replay()
        return self.static_outputs
