"""spear_amd: SPEAR's Block Two-Pass operator and Phalanx layer on AMD MI355X (gfx950).

Mirrors the reference's top-level package (spear/__init__.py:6-9): ``Phalanx``, ``SigmoidA``,
``btp`` and ``__version__``. ``import spear_amd as spear`` is the intended way to switch.
"""

from spear_amd.nn.phalanx import Phalanx, SigmoidA
from spear_amd.ops.btp import btp, btp_log, btp_qkv, phalanx_mix

__version__ = "0.1.0"

__all__ = ["Phalanx", "SigmoidA", "btp", "btp_log", "btp_qkv", "phalanx_mix", "__version__"]
