"""Block Two-Pass (BTP) operator package (spear/ops/btp/__init__.py)."""

from .interface import btp, btp_log

__all__ = ["btp", "btp_log"]
