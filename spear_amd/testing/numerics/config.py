"""Frozen description objects for numerics sweeps (spear/testing/numerics/config.py:16-92).

Only the two ``*_INPUT_DISTRIBUTION`` constants are consumed by the runners; the sweep objects
exist so that configuration files written against the reference keep importing.
"""

from __future__ import annotations

from collections.abc import Sequence
from dataclasses import dataclass, field

import torch


@dataclass(frozen=True)
class DistributionSpec:
    """A sampler name (``normal`` | ``sigmoid_normal`` | ``uniform``) and its parameters."""

    name: str
    params: dict[str, float] = field(default_factory=dict)


@dataclass(frozen=True)
class InputDistributionConfig:
    """How activations and decay coefficients are drawn together."""

    label: str
    activation: DistributionSpec
    coeff: DistributionSpec


@dataclass(frozen=True)
class DimensionSweep:
    name: str
    values: Sequence[int]
    label: str | None = None


@dataclass(frozen=True)
class ReferenceConfig:
    label: str
    runner: str
    coeff_dtype: torch.dtype | None = None
    x_dtype: torch.dtype | None = None


@dataclass(frozen=True)
class NumericsConfig:
    kernel_dtype: torch.dtype
    output_dtype: torch.dtype = torch.float32
    k: int = 2
    base_seed: int = 1234
    samples_per_point: int = 1
    metric: str = "max_abs"
    dimension_sweeps: Sequence[DimensionSweep] = field(default_factory=tuple)
    distributions: Sequence[InputDistributionConfig] = field(default_factory=tuple)
    references: Sequence[ReferenceConfig] = field(default_factory=tuple)


def _dist(label: str, act_std: float, coeff_std: float) -> InputDistributionConfig:
    return InputDistributionConfig(
        label=label,
        activation=DistributionSpec("normal", {"std": act_std}),
        coeff=DistributionSpec("sigmoid_normal", {"std": coeff_std}),
    )


# activations ~ N(0, 1), coefficients ~ sigmoid(N(0, 1))        (config.py:67-71)
DEFAULT_INPUT_DISTRIBUTION = _dist("standard", 1.0, 1.0)
# activations ~ N(0, 1.5), coefficients ~ sigmoid(N(0, 3))      (config.py:73-77)
HEAVY_TAIL_INPUT_DISTRIBUTION = _dist("heavy_tail", 1.5, 3.0)

DEFAULT_DIMENSION_SWEEPS = (
    DimensionSweep("B", (1, 2, 4, 8, 16), label="Batch Size"),
    DimensionSweep("H", (1, 2, 4, 8, 16, 32), label="Heads"),
    DimensionSweep("L", (64, 128, 256, 512, 1024, 2048), label="Sequence Length"),
)

__all__ = [
    "DistributionSpec",
    "InputDistributionConfig",
    "DimensionSweep",
    "ReferenceConfig",
    "NumericsConfig",
    "DEFAULT_INPUT_DISTRIBUTION",
    "HEAVY_TAIL_INPUT_DISTRIBUTION",
    "DEFAULT_DIMENSION_SWEEPS",
]
