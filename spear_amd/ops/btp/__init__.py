"""Block Two-Pass (BTP) operator package (spear/ops/btp/__init__.py)."""

from .interface import btp

__all__ = ["btp"]
