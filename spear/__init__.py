"""The reference's import name over the MI355X implementation: ``import spear`` gives the package
``spear_amd`` under the names the reference's users write (spear/__init__.py:6-9 there):

    from spear import Phalanx, SigmoidA, btp, __version__
    from spear.ops.btp import btp                      from spear.ops.btp.interface import DH, BLK
    from spear.nn.phalanx import Phalanx               from spear.nn.phalanx.inference import step_jagged
    from spear.testing.numerics import ...             import spear._btp   (the compiled binding)

No code lives here: every ``spear.<x>`` is the very module object ``spear_amd.<x>`` (a finder on
``sys.meta_path`` resolves the name, so classes, custom-op registrations and module state exist once),
and ``spear._btp`` is the compiled torch binding ``spear_amd._btp_ext``, which exports the reference's
``forward`` / ``backward`` (csrc/btp/_bindings.cu:240-243).
"""

import importlib
import importlib.abc
import importlib.util
import sys

import spear_amd
from spear_amd import Phalanx, SigmoidA, btp, btp_log, btp_qkv, phalanx_mix
from spear_amd import __version__

__all__ = ["Phalanx", "SigmoidA", "btp", "btp_log", "btp_qkv", "phalanx_mix", "__version__"]


class _AliasLoader(importlib.abc.Loader):
    def __init__(self, target: str):
        self.target = target

    def create_module(self, spec):
        if self.target == "spear_amd._btp_ext":
            from spear_amd import _btp

            module = _btp.load_extension()  # raises with the build instruction if it is not built
        else:
            module = importlib.import_module(self.target)
        self.own_spec = module.__spec__
        return module

    def exec_module(self, module):
        # The module is already initialised; the import system has just stamped the alias's spec on it,
        # which would break later imports under its real name.
        module.__spec__ = self.own_spec


class _AliasFinder(importlib.abc.MetaPathFinder):
    def find_spec(self, fullname, path=None, target=None):
        if not fullname.startswith("spear."):
            return None
        rest = fullname[len("spear."):]
        real = "spear_amd._btp_ext" if rest == "_btp" else "spear_amd." + rest
        if real != "spear_amd._btp_ext" and importlib.util.find_spec(real) is None:
            return None
        return importlib.util.spec_from_loader(fullname, _AliasLoader(real))


if not any(isinstance(f, _AliasFinder) for f in sys.meta_path):
    sys.meta_path.insert(0, _AliasFinder())
