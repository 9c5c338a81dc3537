"""Harness pieces for kernel-vs-reference comparisons.

Counterpart of the reference's ``spear.testing.numerics`` package (spear/testing/numerics/
__init__.py:8-37): every name it exports is exported here, plus the layer helpers of
``.layers``, so its runners and tests read the same against this package.
"""

from . import config as _config
from . import layers as _layers
from . import metrics as _metrics
from . import sampling as _sampling

__all__ = []
for _module, _names in (
    (_config, _config.__all__),
    (_sampling, ("manual_seed", "make_generator", "sample_tensor_from_spec")),
    (_metrics, ("compute_error_metrics", "compute_backward_metrics", "maybe_synchronize")),
    (_layers, ("copy_layer_weights", "compare_layer_parameters", "extract_layer_gradients")),
):
    for _name in _names:
        globals()[_name] = getattr(_module, _name)
        __all__.append(_name)
del _module, _names, _name
