"""Surrogate object -> (kernel id, alpha) for the hip backward kernels.

Same contract as the reference's ``triton_kernel/surrogate_kernel.py:26-34, 98-157``:
resolution is by ``isinstance``; an unsupported surrogate raises ``NotImplementedError``
naming its class; ``alpha`` must be a real scalar (a one-element tensor is accepted).
"""

from __future__ import annotations

import torch

from .. import surrogate

SG_HIP_IDS: dict[type, int] = {
    surrogate.Sigmoid: 0,
    surrogate.ATan: 1,
    surrogate.PiecewiseQuadratic: 2,
    surrogate.PiecewiseExp: 3,
    surrogate.SoftSign: 4,
    surrogate.SuperSpike: 5,
    surrogate.Erf: 6,
}


def resolve_sg_hip_id_and_alpha(surrogate_function) -> tuple[int, float]:
    sg_id = None
    for sg_type, candidate in SG_HIP_IDS.items():
        if isinstance(surrogate_function, sg_type):
            sg_id = candidate
            break
    if sg_id is None:
        names = tuple(t.__name__ for t in SG_HIP_IDS)
        raise NotImplementedError(
            f"hip backend only supports surrogate functions {names}, but got "
            f"{type(surrogate_function).__name__}. Use backend='torch' for other surrogate functions."
        )
    if not hasattr(surrogate_function, "alpha"):
        raise TypeError(
            "hip backend requires surrogate_function.alpha, but got "
            f"{type(surrogate_function).__name__} without 'alpha'."
        )
    alpha = surrogate_function.alpha
    if isinstance(alpha, torch.Tensor):
        if alpha.numel() != 1:
            raise TypeError(
                "surrogate_function.alpha must be a scalar for the hip backend, "
                f"but got tensor with shape={tuple(alpha.shape)}."
            )
        alpha = alpha.item()
    if not isinstance(alpha, (int, float)):
        raise TypeError(
            "surrogate_function.alpha must be a real scalar for the hip backend, "
            f"but got {type(alpha).__name__}."
        )
    return sg_id, float(alpha)
