"""Headline-size checks (B=1024, H=32, L=128 and the long / wide configurations) through
size-independent properties, plus the oracle on a sample of rows."""

import numpy as np
import pytest
import torch

from helpers import BF16_ATOL, BF16_RTOL, F32_ATOL, F32_RTOL, assert_close, f64, make_inputs
from oracle import btp_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _fwd(c, x, k=2, out_dtype=torch.bfloat16):
    from spear_amd import _btp

    B, H, _, L = x.shape
    y = torch.empty(B, H, 16, L, device=DEV, dtype=out_dtype)
    ck = torch.empty(B, H, L // 16, 16, device=DEV, dtype=torch.float32)
    _btp.forward(c, x, y, ck, k, 32, flags=0)
    return y


def _bwd(c, x, g, k=2):
    from spear_amd import _btp

    B, H, _, L = x.shape
    dx = torch.empty_like(x)
    dA = torch.empty(B, H, L, device=DEV, dtype=torch.float32)
    ck = torch.empty(B, H, L // 16, 16, device=DEV, dtype=torch.float32)
    _btp.backward(c, x, g, ck, dx, dA, k, 32)
    return dx, dA


CONFIGS = {
    "c3_B1024_H32_L128": dict(B=1024, H=32, L=128, seed=1234, x_std=0.25, gate="sigmoid"),
    "c4_B16_H64_L8192": dict(B=16, H=64, L=8192, seed=1235, x_std=0.25, gate="sigmoid"),
    "c5_B64_H128_L2048": dict(B=64, H=128, L=2048, seed=1236, x_std=1.0, gate="mixed"),
}


@pytest.mark.parametrize("name", list(CONFIGS))
def test_full_size_properties(name):
    cfg = CONFIGS[name]
    B, H, L = cfg["B"], cfg["H"], cfg["L"]
    print(f"{name}: generating inputs", flush=True)
    coeff, x, dy = make_inputs(B, H, L, cfg["seed"], x_std=cfg["x_std"], gate=cfg["gate"])
    c, xx, g = coeff.to(DEV), x.to(DEV), dy.to(DEV)

    print(f"{name}: forward/backward", flush=True)
    y32 = _fwd(c, xx, out_dtype=torch.float32)
    y16 = _fwd(c, xx)
    dx, dA = _bwd(c, xx, g)
    torch.cuda.synchronize()
    assert torch.isfinite(y32).all() and torch.isfinite(dx.float()).all() and torch.isfinite(dA).all()

    # bf16 output is the rounding of the fp32 output
    assert torch.equal(y16, y32.to(torch.bfloat16))

    # adjoint identity <dy, y> == <dx, x> per (b, h) row; dx is rounded to bf16, hence the tolerance
    lhs = (g.double() * y32.double()).sum(dim=(2, 3))
    rhs = (dx.double() * xx.double()).sum(dim=(2, 3))
    scale = (g.double().abs() * y32.double().abs()).sum(dim=(2, 3))
    assert ((lhs - rhs).abs() <= 4e-3 * scale + 1e-6).all(), "adjoint identity violated"

    # linearity in x: btp(a, 2x) == 2 btp(a, x) exactly (power-of-two scaling commutes with rounding)
    assert torch.equal(_fwd(c, xx * 2, out_dtype=torch.float32), y32 * 2)

    # a block depends on itself and its predecessor only: perturbing block 0 leaves blocks >= 2 alone
    if L >= 48:
        xp = xx.clone()
        xp[..., :16] += 1.0
        yp = _fwd(c, xp, out_dtype=torch.float32)
        assert torch.equal(yp[..., 32:], y32[..., 32:])
        assert not torch.equal(yp[..., :32], y32[..., :32])

    # k = 1 equals running every block on its own
    y_k1 = _fwd(c, xx, k=1, out_dtype=torch.float32)
    blk = L // 16
    cb = c.reshape(B, H, blk, 16).permute(0, 2, 1, 3).reshape(B * blk, H, 16).contiguous()
    xb = xx.reshape(B, H, 16, blk, 16).permute(0, 3, 1, 2, 4).reshape(B * blk, H, 16, 16).contiguous()
    yb = _fwd(cb, xb, out_dtype=torch.float32).reshape(B, blk, H, 16, 16).permute(0, 2, 3, 1, 4).reshape(B, H, 16, L)
    assert torch.equal(y_k1, yb)

    # oracle on a sample of (b, h) rows
    print(f"{name}: oracle on sampled rows", flush=True)
    rng = np.random.default_rng(cfg["seed"])
    bs = rng.integers(0, B, size=6)
    hs = rng.integers(0, H, size=6)
    for b, h in zip(bs, hs):
        a_ = f64(coeff[b : b + 1, h : h + 1])
        x_ = f64(x[b : b + 1, h : h + 1])
        g_ = f64(dy[b : b + 1, h : h + 1])
        assert_close(f64(y32[b : b + 1, h : h + 1]), orc.forward(a_, x_), F32_ATOL, F32_RTOL, f"y32[{b},{h}]")
        assert_close(f64(y16[b : b + 1, h : h + 1]), orc.forward(a_, x_), BF16_ATOL, BF16_RTOL, f"y16[{b},{h}]")
        rdx, rdA = orc.backward(a_, x_, g_)
        assert_close(f64(dx[b : b + 1, h : h + 1]), rdx, BF16_ATOL, BF16_RTOL, f"dx[{b},{h}]")
        assert_close(f64(dA[b : b + 1, h : h + 1]), rdA, F32_ATOL, F32_RTOL, f"dA[{b},{h}]")
