"""Five aggregate error figures shared by all numerics tests
(spear/testing/numerics/metrics.py:25-44): ``max_abs, mean_abs, max_rel, mean_rel, rmse``
with ``rel = |k - r| / (|r| + eps)``, ``eps = 1e-7``, evaluated in float32."""

from __future__ import annotations

import torch

__all__ = ["compute_error_metrics", "compute_backward_metrics", "maybe_synchronize"]


def compute_error_metrics(kernel_out: torch.Tensor, reference_out: torch.Tensor, *, eps: float = 1e-7) -> dict[str, float]:
    got = kernel_out.to(torch.float32)
    want = reference_out.to(torch.float32).to(got.device)
    err = (got - want).abs()
    rel = err / (want.abs() + eps)
    return {
        "max_abs": err.max().item(),
        "mean_abs": err.mean().item(),
        "max_rel": rel.max().item(),
        "mean_rel": rel.mean().item(),
        "rmse": err.square().mean().sqrt().item(),
    }


def compute_backward_metrics(grad_kernel: torch.Tensor, grad_reference: torch.Tensor, *, eps: float = 1e-7) -> dict[str, float]:
    return compute_error_metrics(grad_kernel, grad_reference, eps=eps)


def maybe_synchronize(device: torch.device) -> None:
    if torch.device(device).type == "cuda":
        torch.cuda.synchronize(device)
