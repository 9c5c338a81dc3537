"""Helpers the layer comparisons share: give two layers the same weights, check that they have
them, and snapshot a layer's parameter gradients. Same names and arguments as the reference's
spear/testing/numerics/layers.py:20-52."""

from __future__ import annotations

import torch
import torch.nn as nn

__all__ = ["copy_layer_weights", "compare_layer_parameters", "extract_layer_gradients"]


def copy_layer_weights(source_layer: nn.Module, target_layer: nn.Module) -> None:
    """``target_layer`` takes every parameter and buffer of ``source_layer`` (devices may differ)."""
    target_layer.load_state_dict(source_layer.state_dict())


def compare_layer_parameters(layer1: nn.Module, layer2: nn.Module, *, rtol: float = 1e-5, atol: float = 1e-8) -> bool:
    """True when both layers hold the same entries and every pair is ``allclose``."""
    mine, theirs = layer1.state_dict(), layer2.state_dict()
    if set(mine) != set(theirs):
        return False
    for key, value in mine.items():
        if not torch.allclose(value, theirs[key].to(value.device), rtol=rtol, atol=atol):
            return False
    return True


def extract_layer_gradients(layer: nn.Module) -> dict[str, torch.Tensor]:
    """A detached copy of every parameter's gradient by parameter name; zeros where none has been
    accumulated, so that two layers always yield the same keys."""
    grads: dict[str, torch.Tensor] = {}
    for name, param in layer.named_parameters():
        grads[name] = torch.zeros_like(param) if param.grad is None else param.grad.detach().clone()
    return grads
