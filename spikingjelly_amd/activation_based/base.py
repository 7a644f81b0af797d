"""Step-mode and stateful-module base classes.

Behavioural counterpart of the reference's ``spikingjelly/activation_based/base.py``
(``check_backend_library`` :35-96, ``StepModule`` :99-210, ``MemoryModule`` :313-1125),
written for this package; the one addition is the ``'hip'`` backend, available when
``libsjhip.so`` can be loaded.
"""

from __future__ import annotations

import copy
from typing import Any, Generator, Tuple

import torch
import torch.nn as nn

from ..logger import logger

__all__ = [
    "check_backend_library",
    "StepModule",
    "SingleStepModule",
    "MultiStepModule",
    "MemoryModule",
]


def check_backend_library(backend: str) -> None:
    """Raise ``ImportError`` when the native library behind ``backend`` is missing.

    ``'torch'`` needs nothing.  ``'hip'`` needs ``libsjhip.so`` next to the package
    (reference: base.py:35-96 does the same for cupy / triton / lava).
    """
    if backend == "torch":
        return
    if backend == "hip":
        from .hip_kernel import library

        try:
            library.load()
        except OSError as e:
            raise ImportError(
                "The hip backend needs libsjhip.so; build it with "
                "`make -C spikingjelly_amd/csrc` (hipcc, gfx950)."
            ) from e
        return
    logger.debug("check_backend_library: nothing to check for backend %s", backend)


class StepModule:
    """Mixin giving a module a validated ``step_mode`` ('s' single step, 'm' multi step)."""

    def supported_step_mode(self) -> Tuple[str, ...]:
        return ("s", "m")

    @property
    def step_mode(self) -> str:
        return self._step_mode

    @step_mode.setter
    def step_mode(self, value: str):
        if value not in self.supported_step_mode():
            raise ValueError(
                f'step_mode can only be {self.supported_step_mode()}, but got "{value}"!'
            )
        self._step_mode = value


class SingleStepModule(StepModule):
    def supported_step_mode(self):
        return ("s",)


class MultiStepModule(StepModule):
    def supported_step_mode(self):
        return ("m",)


class MemoryModule(nn.Module, StepModule):
    """``nn.Module`` with named *memories* (state that is reset between samples).

    Memories live in ``self._memories`` (not in ``state_dict``) and are reachable as
    attributes.  ``forward`` materialises the states for the incoming input, calls the
    pure ``*_functional_forward`` and writes the returned states back.
    """

    def __init__(self):
        super().__init__()
        self._memories = {}
        self._memories_rv = {}
        self._backend = "torch"
        self._step_mode = "s"

    # ---- backend -------------------------------------------------------------------
    @property
    def supported_backends(self) -> Tuple[str, ...]:
        return ("torch",)

    @property
    def backend(self) -> str:
        return self._backend

    @backend.setter
    def backend(self, value: str):
        if value not in self.supported_backends:
            raise NotImplementedError(
                f"{value} is not a supported backend of {self._get_name()}!"
            )
        check_backend_library(value)
        self._backend = value

    # ---- functional core -----------------------------------------------------------
    def materialize_states(
        self, inputs: tuple[Any, ...], states: tuple[Any, ...], step_mode: str
    ) -> tuple[Any, ...]:
        return states

    def single_step_functional_forward(
        self, inputs: tuple[torch.Tensor, ...], states: tuple[Any, ...], **kwargs: Any
    ) -> tuple[tuple[torch.Tensor, ...], tuple[Any, ...]]:
        raise NotImplementedError(
            f"{self._get_name()} does not implement single_step_functional_forward."
        )

    def multi_step_functional_forward(
        self, inputs: tuple[torch.Tensor, ...], states: tuple[Any, ...], **kwargs: Any
    ) -> tuple[tuple[torch.Tensor, ...], tuple[Any, ...]]:
        # default: loop the single-step transition over dim 0 and stack the outputs
        per_step = []
        for t in range(inputs[0].shape[0]):
            outputs, states = self.single_step_functional_forward(
                tuple(x[t] for x in inputs), states, **kwargs
            )
            per_step.append(outputs)
        stacked = tuple(torch.stack(seq) for seq in zip(*per_step, strict=True))
        return stacked, states

    def functional_forward(
        self, inputs: tuple[torch.Tensor, ...], states: tuple[Any, ...], **kwargs: Any
    ) -> tuple[tuple[torch.Tensor, ...], tuple[Any, ...]]:
        """Pure forward: never reads or writes ``self._memories``."""
        if self.step_mode == "s":
            states = self.materialize_states(inputs, states, "s")
            return self.single_step_functional_forward(inputs, states, **kwargs)
        if self.step_mode == "m":
            states = self.materialize_states(inputs, states, "m")
            return self.multi_step_functional_forward(inputs, states, **kwargs)
        raise ValueError(self.step_mode)

    def _write_back(self, states: tuple[Any, ...]) -> None:
        for name, value in zip(self._memories, states, strict=True):
            self._memories[name] = value

    def single_step_forward(self, x: torch.Tensor, *args, **kwargs):
        inputs = (x, *args)
        states = self.materialize_states(inputs, tuple(self._memories.values()), "s")
        outputs, states = self.single_step_functional_forward(inputs, states, **kwargs)
        self._write_back(states)
        return outputs[0] if len(outputs) == 1 else outputs

    def multi_step_forward(self, x_seq: torch.Tensor, *args, **kwargs):
        inputs = (x_seq, *args)
        states = self.materialize_states(inputs, tuple(self._memories.values()), "m")
        outputs, states = self.multi_step_functional_forward(inputs, states, **kwargs)
        self._write_back(states)
        return outputs[0] if len(outputs) == 1 else outputs

    def forward(self, *args, **kwargs):
        if self.step_mode == "s":
            return self.single_step_forward(*args, **kwargs)
        if self.step_mode == "m":
            return self.multi_step_forward(*args, **kwargs)
        raise ValueError(self.step_mode)

    def extra_repr(self):
        return f"step_mode={self.step_mode}, backend={self.backend}"

    # ---- memories ------------------------------------------------------------------
    def register_memory(self, name: str, value) -> None:
        assert not hasattr(self, name), f"{name} has been set as a member variable!"
        self._memories[name] = value
        self.set_reset_value(name, value)

    def set_reset_value(self, name: str, value) -> None:
        self._memories_rv[name] = copy.deepcopy(value)

    def get_reset_value(self, name: str) -> Any:
        if name not in self._memories:
            raise KeyError(f"{name} is not a registered memory.")
        if name not in self._memories_rv:
            raise KeyError(f"{name} has no reset value. Call set_reset_value first.")
        return self._memories_rv[name]

    def reset(self) -> None:
        """Restore every memory to its reset value.

        A tensor state whose reset value is a Python scalar goes back to that scalar,
        so the next forward re-materialises it for whatever shape arrives.
        """
        for key, cur in self._memories.items():
            rv = self._memories_rv[key]
            same_kind = (
                isinstance(cur, torch.Tensor)
                and isinstance(rv, torch.Tensor)
                and cur.shape == rv.shape
                and cur.dtype == rv.dtype
                and cur.device == rv.device
            )
            if same_kind:
                try:
                    cur.detach_()  # drop the old graph before the in-place copy
                except RuntimeError:  # views cannot be detached in place
                    self._memories[key] = rv.detach().clone()
                else:
                    cur.copy_(rv)
            elif isinstance(cur, torch.Tensor) and isinstance(rv, (int, float)):
                self._memories[key] = rv
            else:
                self._memories[key] = copy.deepcopy(rv)

    def __getattr__(self, name: str):
        memories = self.__dict__.get("_memories")
        if memories is not None and name in memories:
            return memories[name]
        return super().__getattr__(name)

    def __setattr__(self, name: str, value) -> None:
        memories = self.__dict__.get("_memories")
        if memories is not None and name in memories:
            memories[name] = value
        else:
            super().__setattr__(name, value)

    def __delattr__(self, name):
        if name in self._memories:
            del self._memories[name]
            del self._memories_rv[name]
        else:
            super().__delattr__(name)

    def __dir__(self):
        keys = (
            dir(self.__class__)
            + list(self.__dict__.keys())
            + list(self._parameters.keys())
            + list(self._modules.keys())
            + list(self._buffers.keys())
            + list(self._memories.keys())
        )
        return sorted(k for k in keys if not k[0].isdigit())

    def memories(self) -> Generator:
        yield from self._memories.values()

    def named_memories(self) -> Generator:
        yield from self._memories.items()

    def detach(self) -> None:
        for value in self._memories.values():
            if isinstance(value, torch.Tensor):
                value.detach_()

    def _apply(self, fn):
        for key, value in self._memories.items():
            if isinstance(value, torch.Tensor):
                self._memories[key] = fn(value)
        return super()._apply(fn)

    def _replicate_for_data_parallel(self):
        replica = super()._replicate_for_data_parallel()
        replica._memories = self._memories.copy()
        return replica


# ---- memories of a whole module tree -----------------------------------------------------
def _memory_owners(module: nn.Module, path: Tuple[str, ...] = ()):
    """Pre-order walk of the tree: a module before its children, children in registration order."""
    if isinstance(module, MemoryModule):
        yield path, module
    for child_name, child in module.named_children():
        yield from _memory_owners(child, path + (child_name,))


def named_memories(module: nn.Module, prefix: str = "") -> Generator:
    """``(dotted name, value)`` of every memory below ``module``, the tree-wide counterpart of
    ``named_parameters()``.  Order and naming follow the reference (``base.py:1128-1178``): a
    module's own memories in registration order, then its children's."""
    head = (prefix,) if prefix else ()
    for path, owner in _memory_owners(module):
        for name, value in owner.named_memories():
            yield ".".join(head + path + (name,)), value


def memories(module: nn.Module) -> Generator:
    """Values of :func:`named_memories` (reference ``base.py:1181-1221``)."""
    for _, value in named_memories(module):
        yield value


def extract_memories(module: nn.Module) -> list:
    """Snapshot (a list of references, nothing is cloned) of every memory below ``module``
    (reference ``base.py:1224-1262``)."""
    return [value for _, value in named_memories(module)]


def load_memories(module: nn.Module, memory_list: list) -> None:
    """Inverse of :func:`extract_memories`: assign ``memory_list`` to the memories in the same
    order.  A list of the wrong length raises ``ValueError`` before anything is written
    (reference ``base.py:1265-1312``)."""
    slots = [(owner, name) for _, owner in _memory_owners(module) for name, _ in owner.named_memories()]
    if len(slots) != len(memory_list):
        raise ValueError(
            f"Memory length mismatch: model has {len(slots)} memories but list contains {len(memory_list)}"
        )
    for (owner, name), value in zip(slots, memory_list):
        owner._memories[name] = value


def to_functional_forward(module: nn.Module, fn=None):
    """``f(inputs, states, **kwargs) -> (outputs, new_states)`` for any module tree.

    ``states`` is ordered like :func:`extract_memories`; ``outputs`` is always a tuple.  The module's
    own memories are the same before and after a call, also when the forward raises.  Three routes, as in
    the reference (``base.py:1315-1551``): a single ``MemoryModule`` with a pure ``functional_forward`` of
    its own is called directly; an ``nn.Sequential`` whose direct children own every state and are pure
    threads ``states`` through them without touching a memory (a child's tuple output becomes the next
    child's positional arguments, keyword arguments go to the first child only); every other tree runs its
    ordinary ``forward`` (or ``fn``) between a :func:`load_memories` of ``states`` and a restore of what
    was there.
    """
    owners = [owner for _, owner in _memory_owners(module)]
    n_states = sum(len(owner._memories) for owner in owners)

    def check(states) -> None:
        if len(states) != n_states:
            raise ValueError(f"{module.__class__.__name__} expected {n_states} states, but got {len(states)}.")

    def overrides(owner: MemoryModule, name: str) -> bool:
        return getattr(type(owner), name) is not getattr(MemoryModule, name)

    def is_pure(owner: nn.Module) -> bool:
        return isinstance(owner, MemoryModule) and (
            overrides(owner, "functional_forward")
            or overrides(owner, "single_step_functional_forward")
            or (owner.step_mode == "m" and overrides(owner, "multi_step_functional_forward"))
        )

    def as_tuple(result) -> tuple:
        return tuple(result) if isinstance(result, (tuple, list)) else (result,)

    if fn is None and len(owners) == 1 and owners[0] is module and is_pure(module):

        def direct(inputs, states, **kwargs):
            check(states)
            return module.functional_forward(inputs, states, **kwargs)

        return direct

    if fn is None and isinstance(module, nn.Sequential):
        stages = list(module.children())
        counts = [len(stage._memories) if is_pure(stage) else 0 for stage in stages]

        if sum(counts) == n_states:

            def threaded(inputs, states, **kwargs):
                check(states)
                flowing, new_states, first = tuple(inputs), [], 0
                for stage, count in zip(stages, counts):
                    if count:
                        flowing, out_states = stage.functional_forward(flowing, states[first:first + count], **kwargs)
                        new_states.extend(out_states)
                        first += count
                    else:
                        flowing = as_tuple(stage(*flowing, **kwargs))
                    kwargs = {}
                return tuple(flowing), tuple(new_states)

            return threaded

        def call(*inputs, **kwargs):
            flowing = inputs
            for stage in stages:
                flowing = as_tuple(stage(*flowing, **kwargs))
                kwargs = {}
            return flowing[0] if len(flowing) == 1 else flowing

    else:
        call = module.forward if fn is None else fn

    def swapped(inputs, states, **kwargs):
        check(states)
        saved = extract_memories(module)
        load_memories(module, list(states))
        try:
            outputs = as_tuple(call(*inputs, **kwargs))
            new_states = tuple(extract_memories(module))
        finally:
            load_memories(module, saved)
        return outputs, new_states

    return swapped
