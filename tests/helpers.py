"""Shared input builders and comparison helpers for the BTP tests.

Inputs are always drawn on a CPU generator, so a seed means the same bits on every machine;
the oracle sees the bf16-rounded values promoted to float64 (the protocol of the reference's
gold-standard runner, spear/ops/btp/runners.py:111-116).
"""

from __future__ import annotations

import numpy as np
import torch

# north-star tolerances: |got - ref| <= atol + rtol * |ref|
BF16_ATOL = BF16_RTOL = 2e-2
F32_ATOL = F32_RTOL = 1e-4


def make_inputs(B, H, L, seed, *, x_std=1.0, gate="sigmoid", stress=1.0, dtype=torch.bfloat16):
    """coeff [B,H,L], x [B,H,16,L], dy [B,H,16,L] on the CPU in `dtype` (dy also in that dtype)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = (torch.randn(B, H, 16, L, generator=g) * x_std).to(dtype)
    if gate == "sigmoid":  # sigmoid(N(0, stress)) == exp(-softplus(N(0, stress)))
        coeff = torch.sigmoid(torch.randn(B, H, L, generator=g) * stress)
    elif gate == "mixed":  # per head: near-total forgetting or near-identity (log-space stress)
        forget = torch.rand(B, H, 1, generator=g) < 0.5
        lo = -20.0 + 15.0 * torch.rand(B, H, L, generator=g)
        hi = -1e-4 * torch.rand(B, H, L, generator=g)
        coeff = torch.exp(torch.where(forget, lo, hi))
    elif gate == "ones":
        coeff = torch.ones(B, H, L)
    else:
        raise ValueError(gate)
    coeff = coeff.to(dtype)
    dy = torch.randn(B, H, 16, L, generator=g).to(dtype)
    return coeff, x, dy


def f64(t: torch.Tensor) -> np.ndarray:
    return t.detach().to("cpu", torch.float64).numpy()


def assert_close(got, ref, atol, rtol, what=""):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite values in result"
    err = np.abs(got - ref)
    bound = atol + rtol * np.abs(ref)
    worst = np.argmax(err - bound)
    assert (err <= bound).all(), (
        f"{what}: max |err|={err.max():.3e}; worst excess at flat index {worst}: "
        f"got {got.flat[worst]:.6g} ref {ref.flat[worst]:.6g} bound {bound.flat[worst]:.3e}"
    )


def golden_vectors():
    """The committed closed-form vectors (tests/golden/make_vectors.py): {case: {name: array}} with the
    inputs as [1, H, ...] bfloat16-exact float32 arrays and y / dx / dA per k in float64."""
    import pathlib

    blob = np.load(pathlib.Path(__file__).with_name("golden") / "btp_window_vectors.npz")
    out: dict = {}
    for key in blob.files:
        case, rest = key.split(".", 1)
        out.setdefault(case, {})[rest] = blob[key][None]  # add the batch axis
    return out


def jagged_reference_vectors():
    """Vectors written by tests/golden/make_jagged_vectors.py from the reference's own streaming
    functions: {case: {name: array}}; ``meta`` = (prompt length, block length, decode steps, state.i)."""
    import pathlib

    blob = np.load(pathlib.Path(__file__).with_name("golden") / "jagged_reference_vectors.npz")
    out: dict = {}
    for key in blob.files:
        case, rest = key.split(".", 1)
        out.setdefault(case, {})[rest] = blob[key]
    return out


def layer_reference_vectors():
    """Configuration 1 computed by the reference's own layer on its CPU path
    (tests/golden/make_layer_vectors.py)."""
    import pathlib

    return np.load(pathlib.Path(__file__).with_name("golden") / "layer_reference_vectors.npz")


def config1_layer_and_input(method: str, device="cpu"):
    """The layer and input of configuration 1, drawn exactly as the vectors' generator draws them."""
    from spear_amd import Phalanx

    torch.manual_seed(0)
    layer = Phalanx(dim=512, length=128, method=method, dtype=torch.bfloat16)
    x = torch.randn(8, 128, 512).to(torch.bfloat16)
    return layer.to(device), x.to(device)
