"""Integer-valued LIF neuron (reference ``neuron/ilif.py:17-410``)."""

from __future__ import annotations

from .. import functional, surrogate
from .lif import LIFNode


class ILIFNode(LIFNode):
    """I-LIF (ECCV 2024, *Integer-Valued Training and Spike-Driven Inference Spiking Neural Network*):

        H[t] = (1 - 1/tau) V[t-1] + X[t]
        C[t] = round(clip(H[t] / V_th, 0, D))
        V[t] = H[t] - C[t] V_th

    The charge is ``LIFNode``'s with ``decay_input=False`` and ``v_reset=None``; ``D`` and the rectangular
    straight-through gradient window come from ``surrogate_function``, a spiking ``MultiLevelSpikeCount``.
    The output is the integer count ``C[t]`` in ``{0, ..., D}``, identically in ``train()`` and ``eval()``.
    Both step modes support ``backend='torch'`` and ``backend='hip'`` (the reference offers its Triton kernel
    in multi-step mode only, ``neuron/ilif.py:290-292``).
    """

    def __init__(self, tau: float = 4.0 / 3.0, v_threshold: float = 1.0,
                 surrogate_function: surrogate.MultiLevelSpikeCount = surrogate.MultiLevelSpikeCount(4),
                 detach_reset: bool = False, step_mode: str = "s", backend: str = "torch",
                 store_v_seq: bool = False):
        if not isinstance(surrogate_function, surrogate.MultiLevelSpikeCount) or not surrogate_function.spiking:
            raise ValueError("surrogate_function must be a spiking MultiLevelSpikeCount.")
        super().__init__(tau=tau, decay_input=False, v_threshold=v_threshold, v_reset=None,
                         surrogate_function=surrogate_function, detach_reset=detach_reset, step_mode=step_mode,
                         backend=backend, store_v_seq=store_v_seq)

    def single_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend == "hip":
            count_seq, v, _ = functional.ilif_multi_step_hip(inputs[0].unsqueeze(0), states[0], self.tau,
                                                             self.v_threshold, self.surrogate_function,
                                                             self.detach_reset, False)
            count = count_seq[0]
        elif self.backend == "torch":
            count, v = functional.ilif_step(inputs[0], states[0], self.tau, self.v_threshold,
                                            self.surrogate_function, self.detach_reset)
        else:
            raise ValueError(self.backend)
        return (count,), (v, *states[1:])

    def _hip_multi_step(self, x_seq, v, store_v_seq):
        return functional.ilif_multi_step_hip(x_seq, v, self.tau, self.v_threshold, self.surrogate_function,
                                              self.detach_reset, store_v_seq)
