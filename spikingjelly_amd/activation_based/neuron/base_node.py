"""Common machinery of spiking neuron modules (reference ``neuron/base_node.py:252-485``)."""

from __future__ import annotations

import math
from typing import Optional

import torch

from .. import base, surrogate


# read-only one-element tensors that stand for a constant initial state on the hip backend (see _constant_state)
_CONSTANT_STATES: dict = {}


class BaseNode(base.MemoryModule):
    """Stateful spiking neuron with membrane potential memory ``v``.

    ``v`` starts (and is reset to) the Python float ``v_reset`` (hard reset) or ``0.0`` (soft
    reset, ``v_reset=None``) and becomes a tensor shaped like one time step of the input on the
    first forward.  With ``store_v_seq=True`` a multi-step forward also leaves the per-step
    membrane potentials in ``self.v_seq`` (a plain attribute, not a memory).
    """

    def __init__(self, v_threshold: float = 1.0, v_reset: Optional[float] = 0.0,
                 surrogate_function: surrogate.SurrogateFunctionBase = surrogate.Sigmoid(),
                 detach_reset: bool = False, step_mode="s", backend="torch", store_v_seq: bool = False):
        assert isinstance(v_reset, float) or v_reset is None
        assert isinstance(v_threshold, float)
        assert isinstance(detach_reset, bool)
        super().__init__()
        self.register_memory("v", 0.0 if v_reset is None else v_reset)
        self.v_threshold = v_threshold
        self.v_reset = v_reset
        self.detach_reset = detach_reset
        self.surrogate_function = surrogate_function
        self.step_mode = step_mode
        self.backend = backend
        self.store_v_seq = store_v_seq

    @property
    def store_v_seq(self):
        return self._store_v_seq

    @store_v_seq.setter
    def store_v_seq(self, value: bool):
        self._store_v_seq = value
        self.v_seq = None

    def reset(self):
        super().reset()
        self.v_seq = None

    def extra_repr(self):
        return (f"v_threshold={self.v_threshold}, v_reset={self.v_reset}, detach_reset={self.detach_reset}, "
                f"step_mode={self.step_mode}, backend={self.backend}")

    # ---- helpers shared by IF / LIF / PLIF ---------------------------------------------------------
    def _torch_surrogate(self):
        """Surrogate used by the torch backend: plain Heaviside in eval mode unless the
        surrogate is in primitive (non-spiking) mode (reference neuron/lif.py:252-258)."""
        sg = self.surrogate_function
        if self.training or not getattr(sg, "spiking", True):
            return sg
        return surrogate.heaviside

    def _check_hip_surrogate(self):
        """Kernel backends always fire with Heaviside; a primitive-mode surrogate in eval would
        silently change meaning, so it is rejected (reference neuron/lif.py:318-324)."""
        if not self.training and not getattr(self.surrogate_function, "spiking", True):
            raise NotImplementedError(
                "hip backend only supports spiking surrogate functions. "
                "Use backend='torch' for non-spiking surrogate functions."
            )

    def _hip_multi_step(self, x_seq: torch.Tensor, v: torch.Tensor, store_v_seq: bool):
        """``(spike_seq, v_next, v_seq|None)`` from the hip functional of the concrete neuron."""
        raise NotImplementedError

    def single_step_functional_forward(self, inputs, states, **kwargs):
        raise NotImplementedError(f"{self._get_name()} must implement single_step_functional_forward.")

    def multi_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend == "hip":
            self._check_hip_surrogate()
            spike_seq, v, _ = self._hip_multi_step(inputs[0], states[0], False)
            return (spike_seq,), (v,)
        if self.backend == "torch":
            return super().multi_step_functional_forward(inputs, states, **kwargs)
        raise ValueError(self.backend)

    def multi_step_forward(self, x_seq: torch.Tensor, *args, **kwargs):
        if not self.store_v_seq:
            return super().multi_step_forward(x_seq, *args, **kwargs)
        inputs = (x_seq, *args)
        states = self.materialize_states(inputs, tuple(self._memories.values()), "m")
        if self.backend == "hip":
            self._check_hip_surrogate()
            spike_seq, v, v_seq = self._hip_multi_step(x_seq, states[0], True)
            self.v = v
            self.v_seq = v_seq
            return spike_seq
        # torch backend: step loop that also collects v (reference base_node.py:443-464)
        per_step, v_steps = [], []
        for t in range(x_seq.shape[0]):
            outputs, states = self.single_step_functional_forward(tuple(x[t] for x in inputs), states, **kwargs)
            per_step.append(outputs)
            v_steps.append(states[0])
        self._write_back(states)
        self.v_seq = torch.stack(v_steps)
        outputs = tuple(torch.stack(seq) for seq in zip(*per_step, strict=True))
        return outputs[0] if len(outputs) == 1 else outputs

    def _constant_state(self, x: torch.Tensor, value: float) -> torch.Tensor:
        """The state every neuron starts from, with the shape of ``x`` (reference: ``torch.full_like``,
        neuron/base_node.py:474-475).  The hip kernels read a constant state from a single element, so for that
        backend it is a one-element tensor expanded to the shape (read-only, never written back: the next
        state is the kernel's own output) and no ``[N]`` tensor is filled or read."""
        if self.backend == "hip" and x.is_cuda and x.numel() > 1:
            if torch.compiler.is_compiling() or torch.cuda.is_current_stream_capturing():
                # (memory allocated while a graph is being captured belongs to that graph: not kept)
                return x.new_full((1,) * x.dim(), value).expand(x.shape)
            # one element per (device, dtype, value), made once: a fill launch per neuron and call otherwise
            key = (x.device, x.dtype, float(value), math.copysign(1.0, float(value)))
            one = _CONSTANT_STATES.get(key)
            if one is None:
                # The element outlives this call: it must be an ordinary tensor even when the first call comes under
                # torch.inference_mode() (an inference tensor could not be saved for a later training backward), and
                # its fill must have finished before a call on another stream reads it (made once: the wait is free).
                with torch.inference_mode(False):
                    one = torch.full((1,), value, dtype=x.dtype, device=x.device)
                torch.cuda.current_stream(x.device).synchronize()
                _CONSTANT_STATES[key] = one
            return one.view((1,) * x.dim()).expand(x.shape)
        return torch.full_like(x, value, requires_grad=False)

    def materialize_states(self, inputs, states, step_mode: str):
        x = inputs[0][0] if step_mode == "m" else inputs[0]
        v = states[0]
        if isinstance(v, float):
            v = self._constant_state(x, v)
        elif isinstance(v, torch.Tensor):
            if v.shape != x.shape:  # e.g. batch size changed: start again from the reset value
                v = self._constant_state(x, self.v_reset if self.v_reset is not None else 0.0)
            elif v.dtype != x.dtype or v.device != x.device:
                v = v.to(dtype=x.dtype, device=x.device)
        return (v, *states[1:])
