"""Numerics runners for the BTP operator: seeded inputs, kernel / reference execution and
gradient comparison (counterpart of spear/ops/btp/runners.py:38-187, same function names and
protocols).

Protocol kept from the reference:
  * coefficients may be given as ``[H, L]`` and are broadcast over the batch; the kernel's
    ``dA`` is then summed over the batch before it is compared (runners.py:95-100,147-157);
  * the gold standard is the float64 explicit-product reference evaluated on the *rounded*
    kernel inputs promoted to float64, returned as float32 (runners.py:103-108).

Difference: random numbers are drawn on a CPU generator and copied to the device, so a seed
gives the same inputs on every machine and GPU vendor.
"""

from __future__ import annotations

from collections.abc import Callable

import torch

from spear_amd.testing.numerics import (
    DEFAULT_INPUT_DISTRIBUTION,
    InputDistributionConfig,
    compute_backward_metrics,
    make_generator,
    manual_seed,
    maybe_synchronize,
    sample_tensor_from_spec,
)

from .interface import DH, btp
from .reference import block_two_pass_log, block_two_pass_ref

__all__ = [
    "sample_inputs",
    "run_kernel_forward",
    "run_reference",
    "run_reference_logbtp",
    "compare_backward_gradients",
    "RUNNERS",
    "get_runner",
]


def sample_inputs(
    B: int, H: int, L: int, *, dtype: torch.dtype = torch.bfloat16, device: torch.device | None = None,
    seed: int | None = None, stress_scale: float = 1.0, distribution: InputDistributionConfig | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``(coeff [H, L], x [B, H, 16, L])`` in ``dtype`` on ``device`` (default: the GPU)."""
    device = torch.device(device or ("cuda" if torch.cuda.is_available() else "cpu"))
    if seed is not None:
        manual_seed(seed, device)
    cpu = torch.device("cpu")
    gen = make_generator(cpu, seed)
    dist = distribution or DEFAULT_INPUT_DISTRIBUTION
    x = sample_tensor_from_spec(dist.activation, (B, H, DH, L), dtype=dtype, generator=gen, device=cpu)
    coeff = sample_tensor_from_spec(
        dist.coeff, (H, L), dtype=dtype, generator=gen, device=cpu, scale_multiplier=stress_scale
    )
    return coeff.to(device), x.to(device)


def _broadcast_coeff(coeff: torch.Tensor, batch: int) -> torch.Tensor:
    if coeff.dim() == 2:
        return coeff.unsqueeze(0).expand(batch, -1, -1)
    if coeff.shape[0] == batch:
        return coeff
    raise ValueError("coeff must be [H, L] or [B, H, L]")


def _maybe_compiled(compile: bool, compile_opts: dict | None):
    return torch.compile(btp, **(compile_opts or {})) if compile else btp


def run_kernel_forward(
    coeff: torch.Tensor, x: torch.Tensor, *, k: int = 2, output_dtype: torch.dtype = torch.float32,
    wpb: int | None = None, compile: bool = False, compile_opts: dict | None = None,
) -> torch.Tensor:
    fn = _maybe_compiled(compile, compile_opts)
    return fn(_broadcast_coeff(coeff, x.shape[0]).contiguous(), x, k=k, wpb=wpb, output_dtype=output_dtype)


def run_reference(coeff: torch.Tensor, x: torch.Tensor, BL: int = 16) -> torch.Tensor:
    """float64 explicit-product reference, result as float32."""
    return block_two_pass_ref(_broadcast_coeff(coeff, x.shape[0]).double(), x.double(), BL).float()


def run_reference_logbtp(coeff: torch.Tensor, x: torch.Tensor, BL: int = 16) -> torch.Tensor:
    """Log-space reference in the dtype of its inputs (the training-style CPU path)."""
    return block_two_pass_log(_broadcast_coeff(coeff, x.shape[0]), x, BL).float()


def compare_backward_gradients(
    coeff: torch.Tensor, x: torch.Tensor, *, grad_out: torch.Tensor | None = None, k: int = 2,
    output_dtype: torch.dtype = torch.float32, compile: bool = False, compile_opts: dict | None = None,
) -> dict[str, dict[str, float]]:
    """Error metrics of the kernel's ``d coeff`` and ``dx`` against autograd through the float64
    reference, for the same upstream gradient."""
    if grad_out is None:
        gen = torch.Generator().manual_seed(0)
        grad_out = torch.randn(x.shape, generator=gen).to(device=x.device, dtype=output_dtype)
    else:
        grad_out = grad_out.to(output_dtype)
    B = x.shape[0]
    fn = _maybe_compiled(compile, compile_opts)

    coeff_k = _broadcast_coeff(coeff, B).contiguous().clone().detach().requires_grad_(True)
    x_k = x.clone().detach().requires_grad_(True)
    torch.autograd.backward(fn(coeff_k, x_k, k=k, output_dtype=output_dtype), grad_out)
    grad_coeff_k = coeff_k.grad.detach()
    if coeff.dim() == 2:
        grad_coeff_k = grad_coeff_k.sum(dim=0)  # the reference gradient has the un-broadcast shape

    coeff_r = coeff.clone().detach().requires_grad_(True)
    x_r = x.clone().detach().requires_grad_(True)
    (run_reference(coeff_r, x_r).to(output_dtype) * grad_out).sum().backward()
    maybe_synchronize(x.device)
    return {
        "coeff": compute_backward_metrics(grad_coeff_k, coeff_r.grad.detach()),
        "x": compute_backward_metrics(x_k.grad.detach(), x_r.grad.detach()),
    }


RUNNERS: dict[str, Callable[..., torch.Tensor]] = dict(
    kernel=run_kernel_forward, reference_logbtp=run_reference_logbtp, reference=run_reference
)


def get_runner(name: str) -> Callable[..., torch.Tensor]:
    try:
        return RUNNERS[name]
    except KeyError:
        raise ValueError(f"Unknown BTP runner '{name}'") from None
