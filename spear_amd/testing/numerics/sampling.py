"""Seeded samplers (spear/testing/numerics/sampling.py:23-66).

Unlike the reference, ``device`` may be the CPU: a CPU generator gives the same bits on every
machine, which is what makes seeded cases comparable between a CPU oracle and a GPU kernel.
"""

from __future__ import annotations

from collections.abc import Iterable

import torch

from .config import DistributionSpec

__all__ = ["manual_seed", "make_generator", "sample_tensor_from_spec"]


def manual_seed(seed: int, device: torch.device) -> None:
    torch.manual_seed(seed)
    if torch.device(device).type == "cuda":
        torch.cuda.manual_seed_all(seed)


def make_generator(device: torch.device, seed: int | None = None) -> torch.Generator:
    gen = torch.Generator(device=device)
    if seed is not None:
        gen.manual_seed(seed)
    return gen


def sample_tensor_from_spec(
    spec: DistributionSpec,
    shape: Iterable[int] | tuple[int, ...],
    *,
    dtype: torch.dtype,
    generator: torch.Generator,
    device: torch.device,
    scale_multiplier: float = 1.0,
) -> torch.Tensor:
    """Draw in float32 on ``device`` and cast to ``dtype`` last, so the rounding is the only
    difference between dtypes."""
    shape = tuple(shape)
    kind = spec.name.lower()

    def _randn() -> torch.Tensor:
        return torch.randn(shape, generator=generator, device=device, dtype=torch.float32)

    if kind == "normal":
        out = _randn() * (spec.params.get("std", 1.0) * scale_multiplier)
    elif kind == "sigmoid_normal":
        out = torch.sigmoid(_randn() * (spec.params.get("std", 1.0) * scale_multiplier))
    elif kind == "uniform":
        out = torch.empty(shape, device=device, dtype=torch.float32)
        out.uniform_(spec.params.get("low", 0.0), spec.params.get("high", 1.0), generator=generator)
    else:
        raise ValueError(f"Unsupported distribution '{spec.name}'")
    return out.to(dtype)
