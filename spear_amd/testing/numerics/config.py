"""Record types that describe numerics sweeps: which distributions inputs are drawn from, which
dimensions are swept, which reference a kernel is compared with.

Counterpart of the reference's spear/testing/numerics/config.py:16-92: the same five frozen record
types (names, field order, defaults) and the same three constants, so that configuration written
against the reference keeps importing. Only the two ``*_INPUT_DISTRIBUTION`` constants are consumed
by this package's runners.
"""

from __future__ import annotations

import dataclasses
from collections.abc import Sequence

import torch

_EMPTY = dataclasses.field(default_factory=tuple)


def _record(name: str, doc: str, *fields):
    """A frozen dataclass from ``(field, type[, default])`` rows."""
    rows = []
    for row in fields:
        if len(row) == 2:
            rows.append(row)
        else:
            default = row[2]
            spec = default if isinstance(default, dataclasses.Field) else dataclasses.field(default=default)
            rows.append((row[0], row[1], spec))
    cls = dataclasses.make_dataclass(name, rows, frozen=True)
    cls.__doc__ = doc
    cls.__module__ = __name__
    return cls


DistributionSpec = _record(
    "DistributionSpec", "A sampler name (normal | sigmoid_normal | uniform) and its parameters.",
    ("name", str), ("params", "dict[str, float]", dataclasses.field(default_factory=dict)),
)
InputDistributionConfig = _record(
    "InputDistributionConfig", "How activations and decay coefficients are drawn together.",
    ("label", str), ("activation", DistributionSpec), ("coeff", DistributionSpec),
)
DimensionSweep = _record(
    "DimensionSweep", "The values one tensor dimension takes in a sweep.",
    ("name", str), ("values", Sequence[int]), ("label", "str | None", None),
)
ReferenceConfig = _record(
    "ReferenceConfig", "A reference runner and the dtypes it is fed.",
    ("label", str), ("runner", str), ("coeff_dtype", "torch.dtype | None", None), ("x_dtype", "torch.dtype | None", None),
)
NumericsConfig = _record(
    "NumericsConfig", "One numerics sweep: kernel dtypes, seeds, metric, and what is swept against what.",
    ("kernel_dtype", torch.dtype), ("output_dtype", torch.dtype, torch.float32), ("k", int, 2), ("base_seed", int, 1234),
    ("samples_per_point", int, 1), ("metric", str, "max_abs"),
    ("dimension_sweeps", Sequence[DimensionSweep], _EMPTY),
    ("distributions", Sequence[InputDistributionConfig], dataclasses.field(default_factory=tuple)),
    ("references", Sequence[ReferenceConfig], dataclasses.field(default_factory=tuple)),
)


def _gaussian_inputs(label: str, act_std: float, coeff_std: float):
    """Activations ~ N(0, act_std); coefficients ~ sigmoid(N(0, coeff_std))."""
    return InputDistributionConfig(
        label=label,
        activation=DistributionSpec("normal", {"std": act_std}),
        coeff=DistributionSpec("sigmoid_normal", {"std": coeff_std}),
    )


DEFAULT_INPUT_DISTRIBUTION = _gaussian_inputs("standard", 1.0, 1.0)        # config.py:67-71
HEAVY_TAIL_INPUT_DISTRIBUTION = _gaussian_inputs("heavy_tail", 1.5, 3.0)   # config.py:73-77

DEFAULT_DIMENSION_SWEEPS = tuple(
    DimensionSweep(axis, values, label=label)
    for axis, label, values in (
        ("B", "Batch Size", (1, 2, 4, 8, 16)),
        ("H", "Heads", (1, 2, 4, 8, 16, 32)),
        ("L", "Sequence Length", (64, 128, 256, 512, 1024, 2048)),
    )
)

__all__ = [
    "DistributionSpec", "InputDistributionConfig", "DimensionSweep", "ReferenceConfig", "NumericsConfig",
    "DEFAULT_INPUT_DISTRIBUTION", "HEAVY_TAIL_INPUT_DISTRIBUTION", "DEFAULT_DIMENSION_SWEEPS",
]
