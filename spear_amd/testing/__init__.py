"""Test-support utilities that ship with the package (samplers, error metrics, weight helpers)."""

from . import numerics

__all__ = ["numerics"]
