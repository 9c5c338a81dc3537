"""Harness pieces for kernel-vs-reference comparisons.

Counterpart of the reference's ``spear.testing.numerics`` package (spear/testing/numerics/
__init__.py:8-37): same exported names, so its runners and tests read the same here.
"""

from .config import (
    DEFAULT_DIMENSION_SWEEPS,
    DEFAULT_INPUT_DISTRIBUTION,
    HEAVY_TAIL_INPUT_DISTRIBUTION,
    DimensionSweep,
    DistributionSpec,
    InputDistributionConfig,
    NumericsConfig,
    ReferenceConfig,
)
from .layers import compare_layer_parameters, copy_layer_weights, extract_layer_gradients
from .metrics import compute_backward_metrics, compute_error_metrics, maybe_synchronize
from .sampling import make_generator, manual_seed, sample_tensor_from_spec

__all__ = [
    "DistributionSpec",
    "InputDistributionConfig",
    "DimensionSweep",
    "ReferenceConfig",
    "NumericsConfig",
    "DEFAULT_INPUT_DISTRIBUTION",
    "HEAVY_TAIL_INPUT_DISTRIBUTION",
    "DEFAULT_DIMENSION_SWEEPS",
    "manual_seed",
    "make_generator",
    "sample_tensor_from_spec",
    "compute_error_metrics",
    "compute_backward_metrics",
    "maybe_synchronize",
    "copy_layer_weights",
    "compare_layer_parameters",
    "extract_layer_gradients",
]
