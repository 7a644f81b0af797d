"""Shared input generators and comparison helpers for the tests."""

from __future__ import annotations

import json
import os

import numpy as np
import torch

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def seeded_randn(shape, seed: int, mean: float = 0.0, std: float = 1.0, dtype=torch.float32) -> torch.Tensor:
    """CPU tensor ~ N(mean, std) from a fixed seed, the way the benchmark configs define inputs."""
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=dtype) * std + mean


def seeded_rand(shape, seed: int, scale: float = 1.0) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return torch.rand(shape, generator=g, dtype=torch.float32) * scale


def load_dyadic():
    with open(os.path.join(GOLDEN_DIR, "dyadic_4x4.json")) as f:
        return json.load(f)


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Bit-pattern equality (distinguishes -0.0 from 0.0, equates identical NaNs)."""
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    a = a.detach().cpu().contiguous()
    b = b.detach().cpu().contiguous()
    view = {4: torch.int32, 2: torch.int16, 1: torch.uint8}[a.element_size()]
    return torch.equal(a.view(view), b.view(view))


def max_rel_err(actual: torch.Tensor, expected: torch.Tensor, floor: float = 1e-6) -> float:
    a = actual.detach().double().cpu()
    e = expected.detach().double().cpu()
    return float(((a - e).abs() / e.abs().clamp_min(floor)).max())


def require_device_memory(gib: int) -> None:
    """Skip a full-size test on a small card; on an MI355X-class card (192 GiB or more in total) too little free
    memory is a failure, so that a run there cannot silently drop the benchmark-shape tests."""
    import pytest

    free, total = torch.cuda.mem_get_info()
    if free >= gib * (1 << 30):
        return
    message = f"needs {gib} GiB of free device memory, {free / (1 << 30):.1f} of {total / (1 << 30):.1f} GiB are free"
    if total >= 192 * (1 << 30):
        pytest.fail(message)
    pytest.skip(message)


def np_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().to(torch.float32).numpy()
