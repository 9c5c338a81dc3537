"""Weight-copy and gradient-collection helpers for layer comparisons
(spear/testing/numerics/layers.py:20-52)."""

from __future__ import annotations

import torch
import torch.nn as nn

__all__ = ["copy_layer_weights", "compare_layer_parameters", "extract_layer_gradients"]


def copy_layer_weights(source_layer: nn.Module, target_layer: nn.Module) -> None:
    target_layer.load_state_dict(source_layer.state_dict())


def compare_layer_parameters(layer1: nn.Module, layer2: nn.Module, *, rtol: float = 1e-5, atol: float = 1e-8) -> bool:
    sd1, sd2 = layer1.state_dict(), layer2.state_dict()
    if sd1.keys() != sd2.keys():
        return False
    return all(torch.allclose(sd1[k], sd2[k].to(sd1[k].device), rtol=rtol, atol=atol) for k in sd1)


def extract_layer_gradients(layer: nn.Module) -> dict[str, torch.Tensor]:
    return {
        name: (p.grad.detach().clone() if p.grad is not None else torch.zeros_like(p))
        for name, p in layer.named_parameters()
    }
