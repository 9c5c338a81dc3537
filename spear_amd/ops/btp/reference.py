"""PyTorch statement of the Block Two-Pass operator (device-agnostic, differentiable).

These functions back ``Phalanx(method="pytorch")`` / ``method="pytorch_linspace"`` and the numerics
runners. They are explicit, user-selected methods: :func:`spear_amd.ops.btp.btp` never routes here,
and raises when the HIP library is missing instead of falling back.

Same names, argument order and tensor layouts as the reference module
(spear/ops/btp/reference.py):

============================================  =====================================
this module                                   reference lines
============================================  =====================================
``segsum`` / ``construct_L_exp_segsum_log``    spear/ops/btp/reference.py:21-33
``segsum_stable`` / ``..._log_stable``         spear/ops/btp/reference.py:38-52
``construct_L_ref``                            spear/ops/btp/reference.py:55-77
``construct_L_masked_cumprod``                 spear/ops/btp/reference.py:79-90
``construct_L_cumprod_ratio``                  spear/ops/btp/reference.py:92-102
``block_two_pass``                             spear/ops/btp/reference.py:105-139
``block_two_pass_{ref,log,linspace}``          spear/ops/btp/reference.py:142-152
============================================  =====================================

Every ``construct_L_*`` maps ``a[..., T]`` to ``L[..., T, T]`` with
``L[i, j] = a[j+1] * ... * a[i]`` for ``i > j``, ``1`` on the diagonal and ``0`` above it.
"""

from __future__ import annotations

import torch

__all__ = ["block_two_pass_ref", "block_two_pass_log", "block_two_pass_linspace"]


def _tri(T: int, device, diagonal: int) -> torch.Tensor:
    return torch.ones(T, T, dtype=torch.bool, device=device).tril(diagonal)


def segsum(x: torch.Tensor) -> torch.Tensor:
    """Difference-of-prefix-sums segment sum: ``S[i, j] = cs[i] - cs[j]`` (``-inf`` above the
    diagonal). Cheap but cancels badly for long or steep segments; kept for comparison."""
    T = x.shape[-1]
    cs = x.cumsum(-1)
    diff = cs.unsqueeze(-1) - cs.unsqueeze(-2)
    return diff.masked_fill(~_tri(T, x.device, 0), float("-inf"))


def construct_L_exp_segsum_log(a: torch.Tensor) -> torch.Tensor:
    return segsum(a.log()).exp()


def segsum_stable(x: torch.Tensor) -> torch.Tensor:
    """``S[i, j] = x[j+1] + ... + x[i]`` accumulated term by term down each column, so two large
    prefixes are never subtracted."""
    T = x.shape[-1]
    by_row = x.unsqueeze(-1).expand(*x.shape, T)  # by_row[..., i, j] = x[..., i]
    strictly_below = _tri(T, x.device, -1)
    running = torch.where(strictly_below, by_row, torch.zeros((), dtype=x.dtype, device=x.device)).cumsum(-2)
    return running.masked_fill(~_tri(T, x.device, 0), float("-inf"))


def construct_L_exp_segsum_log_stable(a: torch.Tensor) -> torch.Tensor:
    return segsum_stable(a.log()).exp()


def construct_L_ref(a: torch.Tensor) -> torch.Tensor:
    """Explicit products in float64, one sub-diagonal at a time:
    ``L[i, i-g] = a[i-g+1] * L[i, i-g+1]``. The result is cast back to ``a.dtype``."""
    T = a.shape[-1]
    a64 = a.double()
    eye = torch.eye(T, dtype=torch.float64, device=a.device)
    out = eye.expand(*a.shape[:-1], T, T).clone()
    band = torch.ones_like(a64)  # band[..., i] = L[i, i-g+1] for the current g
    rows = torch.arange(T, device=a.device)
    for g in range(1, T):
        # factor entering the product when the column moves left by one: a[i-g+1]
        shifted = torch.ones_like(a64)
        shifted[..., g:] = a64[..., 1 : T - g + 1]
        band = band * shifted
        i = rows[g:]
        out[..., i, i - g] = band[..., g:]
    return out.to(a.dtype)


def construct_L_masked_cumprod(x: torch.Tensor) -> torch.Tensor:
    """Linear-space construction: running product down each column of the strictly-lower part."""
    T = x.shape[-1]
    by_row = x.unsqueeze(-1).expand(*x.shape, T)
    one = torch.ones((), dtype=x.dtype, device=x.device)
    zero = torch.zeros((), dtype=x.dtype, device=x.device)
    prod = torch.where(_tri(T, x.device, -1), by_row, one).cumprod(-2)
    return torch.where(_tri(T, x.device, 0), prod, zero)


def construct_L_cumprod_ratio(x: torch.Tensor) -> torch.Tensor:
    """Ratio of prefix products (unstable once a prefix underflows); kept for comparison."""
    p = x.cumprod(-1)
    num, den = p.unsqueeze(-1), p.unsqueeze(-2)
    ratio = torch.where(den != 0, num / den, torch.zeros_like(num))
    return ratio.masked_fill(~_tri(x.shape[-1], x.device, 0), 0.0)


def block_two_pass(a: torch.Tensor, u: torch.Tensor, L_constructor, BL: int = 16) -> torch.Tensor:
    """Two passes over blocks of ``BL`` steps.

    a: ``[B, H, N]`` decay coefficients; u: ``[B, H, DH, N]`` inputs; returns ``[B, H, DH, N]``.

    Pass 1 contracts every block with its own decay matrix (zero initial state). Pass 2 adds,
    to every block but the first, the previous block's *local* last row scaled by the inclusive
    prefix product of the current block -- one hop only, the carry is not chained further.
    """
    B, H, DH, N = u.shape
    NB = N // BL
    ab = a.reshape(B, H, NB, BL)
    ub = u.reshape(B, H, DH, NB, BL).transpose(2, 3)  # [B, H, NB, DH, BL(j)]

    Lm = L_constructor(ab)  # [B, H, NB, BL(i), BL(j)]
    v = ub @ Lm.transpose(-1, -2)  # [B, H, NB, DH, BL(i)]

    if NB > 1:
        prefix = ab[:, :, 1:, :1] * Lm[:, :, 1:, :, 0]  # a_0 * L[i, 0] = inclusive prefix product
        prev_last = v[:, :, :-1, :, -1]  # [B, H, NB-1, DH]
        hop = prev_last.unsqueeze(-1) * prefix.unsqueeze(-2)
        v = torch.cat([v[:, :, :1], v[:, :, 1:] + hop], dim=2)

    return v.transpose(2, 3).reshape(B, H, DH, N)


def block_two_pass_ref(a: torch.Tensor, u: torch.Tensor, BL: int = 16) -> torch.Tensor:
    assert u.dtype == a.dtype == torch.float64, "u and a must be float64"
    return block_two_pass(a, u, construct_L_ref, BL)


def block_two_pass_log(a: torch.Tensor, u: torch.Tensor, BL: int = 16) -> torch.Tensor:
    return block_two_pass(a, u, construct_L_exp_segsum_log_stable, BL)


def block_two_pass_linspace(a: torch.Tensor, u: torch.Tensor, BL: int = 16) -> torch.Tensor:
    return block_two_pass(a, u, construct_L_masked_cumprod, BL)
