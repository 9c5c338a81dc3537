"""Block Two-Pass (BTP) operator package (spear/ops/btp/__init__.py)."""

from .fused import btp_qkv, phalanx_mix
from .interface import btp, btp_log

__all__ = ["btp", "btp_log", "btp_qkv", "phalanx_mix"]
