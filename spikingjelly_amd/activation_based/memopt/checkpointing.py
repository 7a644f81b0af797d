"""Input-compressed gradient checkpointing: the training-side consumer of the spike compressors.

Counterpart of the reference's ``memopt/checkpointing.py`` (``InputCompressedGC`` :129-201,
``input_compressed_gc`` :204-282, ``to_gc_function`` :285-371, ``GCContainer`` :374-474, ``TCGCContainer`` :477-602).
A checkpointed segment keeps only its *input* for the backward pass, and keeps it compressed: with a
``BitSpikeCompressor`` a binary spike tensor on the GPU is held as one bit per spike (packed and unpacked by this
library's HIP kernels on the current stream, no host synchronisation).  The forward runs once without a graph; the
backward decompresses the input, runs the forward again with a graph under the forward's autocast and random-number
state, and backpropagates through that.

A segment with memories (spiking neurons) runs through :func:`base.to_functional_forward`: its states enter and leave
the checkpointed function as ordinary arguments and results, so state gradients flow between calls (and between the
temporal chunks of :class:`TCGCContainer`).
"""

from __future__ import annotations

import contextlib
import functools
import threading
from typing import Any, Callable, Optional

import torch
import torch.nn as nn

from ...logger import logger
from .. import base
from .compress import BaseSpikeCompressor, NullSpikeCompressor

__all__ = [
    "in_gc_1st_forward",
    "query_autocast",
    "InputCompressedGC",
    "input_compressed_gc",
    "to_gc_function",
    "GCContainer",
    "TCGCContainer",
]

_per_thread = threading.local()


@contextlib.contextmanager
def _gc_1st_forward():
    """Marks the graph-free first forward of a checkpointed segment for this thread; nests."""
    depth = getattr(_per_thread, "first_forward_depth", 0)
    _per_thread.first_forward_depth = depth + 1
    try:
        yield
    finally:
        _per_thread.first_forward_depth = depth


def in_gc_1st_forward() -> bool:
    """True inside the first (graph-free) forward of a checkpointed segment on the calling thread."""
    return getattr(_per_thread, "first_forward_depth", 0) > 0


def query_autocast() -> tuple[str, torch.dtype, bool]:
    """``(device_type, dtype, enabled)`` of the active autocast; ``("cpu", cpu autocast dtype, False)`` if none."""
    for device_type in ("cuda", "cpu"):
        if torch.is_autocast_enabled(device_type):
            return device_type, torch.get_autocast_dtype(device_type), True
    return "cpu", torch.get_autocast_dtype("cpu"), False


def _separate_args(*args) -> tuple[list, list, list]:
    """``(args with every tensor replaced by None, the tensors, their positions)``."""
    plain, tensors, positions = [], [], []
    for position, arg in enumerate(args):
        if torch.is_tensor(arg):
            plain.append(None)
            tensors.append(arg)
            positions.append(position)
        else:
            plain.append(arg)
    return plain, tensors, positions


def _combine_args(input_args, tensor_args, tensor_args_indices) -> list:
    """Inverse of :func:`_separate_args` (fills ``input_args`` in place and returns it)."""
    for tensor, position in zip(tensor_args, tensor_args_indices):
        input_args[position] = tensor
    return input_args


def _cuda_devices_of(tensors) -> list[int]:
    return sorted({t.device.index for t in tensors if t.device.type == "cuda"})


class InputCompressedGC(torch.autograd.Function):
    """``outputs = f_forward(x_seq, *args)`` keeping ``x_compressor.compress(x_seq)`` and ``args`` for the backward."""

    @staticmethod
    def forward(ctx, f_forward: Callable, x_compressor: BaseSpikeCompressor, x_seq: torch.Tensor, *args):
        ctx.f_forward = f_forward
        ctx.x_compressor = x_compressor
        ctx.x_seq_shape = x_seq.shape
        ctx.autocast = query_autocast()
        ctx.plain_args, kept, ctx.tensor_positions = _separate_args(x_compressor.compress(x_seq), *args)
        ctx.save_for_backward(*kept)
        # random-number state of the forward: the host generator and the generators of the GPUs the arguments live on
        ctx.rng_devices = _cuda_devices_of([x_seq, *kept])
        ctx.rng_cpu = torch.get_rng_state()
        ctx.rng_cuda = [torch.cuda.get_rng_state(d) for d in ctx.rng_devices]
        with _gc_1st_forward(), torch.no_grad():
            return f_forward(x_seq, *args)

    @staticmethod
    def backward(ctx, *grad_outputs):
        grads: list = [None] * (2 + len(ctx.plain_args))
        if not any(ctx.needs_input_grad):
            return tuple(grads)
        x_packed, *args = _combine_args(list(ctx.plain_args), ctx.saved_tensors, ctx.tensor_positions)
        device_type, dtype, enabled = ctx.autocast
        with torch.enable_grad(), torch.autocast(device_type, dtype, enabled):
            # (the reference always asks for the input's gradient; it is only computed here when somebody wants it)
            x_seq = ctx.x_compressor.decompress(x_packed, ctx.x_seq_shape).detach().requires_grad_(bool(ctx.needs_input_grad[2]))
            for i, wanted in enumerate(ctx.needs_input_grad[3:]):
                if torch.is_tensor(args[i]):
                    args[i] = args[i].detach().requires_grad_(wanted and args[i].requires_grad)
            with torch.random.fork_rng(ctx.rng_devices):
                torch.set_rng_state(ctx.rng_cpu)
                for device, state in zip(ctx.rng_devices, ctx.rng_cuda):
                    torch.cuda.set_rng_state(state, device)
                outputs = ctx.f_forward(x_seq, *args)
        if torch.is_tensor(outputs):
            outputs = (outputs,)
        # outputs that carry no graph (integer results, untouched pass-through values) take no gradient
        pairs = [(o, g) for o, g in zip(outputs, grad_outputs) if torch.is_tensor(o) and o.requires_grad and g is not None]
        if pairs:
            torch.autograd.backward([o for o, _ in pairs], [g for _, g in pairs])
        if ctx.needs_input_grad[2]:
            grads[2] = x_seq.grad
        for i, arg in enumerate(args):
            if ctx.needs_input_grad[3 + i] and torch.is_tensor(arg):
                grads[3 + i] = arg.grad
        return tuple(grads)


def input_compressed_gc(f_forward: Callable, x_compressor: BaseSpikeCompressor, x_seq: torch.Tensor, *args):
    """Gradient checkpointing of ``f_forward(x_seq, *args)`` with ``x_seq`` kept compressed.

    ``x_seq`` is typically a spike tensor; ``args`` may mix tensors and other values.  ``f_forward`` must not depend on
    anything that changes between the forward and the backward except the random-number state, which is replayed.
    """
    return InputCompressedGC.apply(f_forward, x_compressor, x_seq, *args)


def to_gc_function(x_compressor: BaseSpikeCompressor, f_forward: Optional[Callable] = None):
    """``f_forward`` wrapped in :func:`input_compressed_gc`; without ``f_forward``, a decorator that does so."""

    def wrap(fn: Callable) -> Callable:
        @functools.wraps(fn)
        def checkpointed(x_seq, *args):
            return input_compressed_gc(fn, x_compressor, x_seq, *args)

        return checkpointed

    return wrap if f_forward is None else wrap(f_forward)


class GCContainer(nn.Sequential):
    """An ``nn.Sequential`` that runs as one checkpointed segment whose first input is kept compressed.

    ``x_compressor=None`` keeps the input as it is (``NullSpikeCompressor``).  The children may hold memories.
    """

    def __init__(self, x_compressor: Optional[BaseSpikeCompressor], *args):
        super().__init__(*args)
        self.x_compressor = NullSpikeCompressor() if x_compressor is None else x_compressor
        self.num_states = len(list(base.memories(self)))
        self.f_forward = base.to_functional_forward(self)

    # the functional forward is a closure over this module: rebuilt instead of pickled or deep-copied
    def __getstate__(self) -> dict:
        state = dict(super().__getstate__())
        state.pop("f_forward", None)
        return state

    def __setstate__(self, state: dict) -> None:
        super().__setstate__(state)
        self.f_forward = base.to_functional_forward(self)

    def super_forward(self, *inputs: Any) -> Any:
        """``nn.Sequential.forward`` with a child's tuple result spread over the next child's arguments."""
        flowing = inputs
        for child in self:
            result = child(*flowing)
            flowing = tuple(result) if isinstance(result, (tuple, list)) else (result,)
        return flowing[0] if len(flowing) == 1 else flowing

    def _needs_anchor(self, *values) -> bool:
        """The segment's parameters are not arguments of the checkpointed function, so when no argument carries a graph
        (the first segment of a network fed with data) its outputs would be leaves and its parameters would get no
        gradient: the reference, like ``torch.utils.checkpoint`` in its re-entrant form, has that limitation.  Here an
        empty tensor that requires a gradient rides along as one more argument in that case."""
        if not torch.is_grad_enabled() or any(torch.is_tensor(v) and v.requires_grad for v in values):
            return False
        return any(p.requires_grad for p in self.parameters())

    def stateless_forward(self, x: torch.Tensor, *args: Any) -> Any:
        if self._needs_anchor(x, *args):
            anchor = x.new_zeros((0,), dtype=torch.float32).requires_grad_()
            return input_compressed_gc(lambda x_, *rest: self.super_forward(x_, *rest[:-1]), self.x_compressor, x, *args,
                                       anchor)
        return input_compressed_gc(self.super_forward, self.x_compressor, x, *args)

    def stateful_forward(self, x: torch.Tensor, *args: Any) -> Any:
        n_inputs, n_states = 1 + len(args), self.num_states
        states = base.extract_memories(self)
        anchor = ((x.new_zeros((0,), dtype=torch.float32).requires_grad_(),) if self._needs_anchor(x, *args, *states)
                  else ())

        def with_explicit_states(*flat):
            if anchor:
                flat = flat[:-1]
            outputs, new_states = self.f_forward(tuple(flat[:n_inputs]), tuple(flat[n_inputs:]))
            return (*outputs, *new_states)

        flat = input_compressed_gc(with_explicit_states, self.x_compressor, x, *args, *states, *anchor)
        base.load_memories(self, flat[-n_states:])
        outputs = flat[:-n_states]
        return outputs[0] if len(outputs) == 1 else outputs

    def forward(self, x, *args):
        return self.stateful_forward(x, *args) if self.num_states else self.stateless_forward(x, *args)

    def extra_repr(self) -> str:
        return f"x_compressor={self.x_compressor.__class__.__name__},"


class TCGCContainer(GCContainer):
    """A :class:`GCContainer` applied to ``n_chunk`` consecutive pieces of the time axis, one checkpoint each.

    The first ``n_seq_inputs`` arguments are sequences ``[T, ...]`` split along ``T`` (``torch.tensor_split``: the
    leading chunks take the remainder); the others are passed to every chunk.  Each of the ``n_outputs`` results is
    concatenated along ``T``.  Memories carry from one chunk to the next.
    """

    def __init__(self, x_compressor: Optional[BaseSpikeCompressor], *args, n_chunk: int = 1, n_seq_inputs: int = 1,
                 n_outputs: int = 1):
        super().__init__(x_compressor, *args)
        self.n_chunk = n_chunk
        self.n_seq_inputs = n_seq_inputs
        self.n_outputs = n_outputs

    def forward(self, x_seq: torch.Tensor, *args):
        T = x_seq.shape[0]
        n_chunk = min(self.n_chunk, T)
        if n_chunk != self.n_chunk:
            logger.warning("TCGCContainer received n_chunk=%d for sequence length T=%d; using n_chunk=%d.",
                           self.n_chunk, T, n_chunk)
        sequences = (x_seq,) + tuple(args[: self.n_seq_inputs - 1])
        shared = tuple(args[self.n_seq_inputs - 1:])
        pieces = [torch.tensor_split(seq, n_chunk, dim=0) for seq in sequences]
        collected: list[list] = [[] for _ in range(self.n_outputs)]
        for chunk in range(n_chunk):
            results = super().forward(*(piece[chunk] for piece in pieces), *shared)
            if not isinstance(results, tuple):
                results = (results,)
            for slot, result in zip(collected, results):
                slot.append(result)
        joined = [torch.cat(slot, dim=0) for slot in collected]
        return joined[0] if len(joined) == 1 else tuple(joined)

    def extra_repr(self) -> str:
        return (f"x_compressor={self.x_compressor.__class__.__name__}, n_chunk={self.n_chunk}, "
                f"n_seq_inputs={self.n_seq_inputs}, n_seq_outputs={self.n_outputs}")
