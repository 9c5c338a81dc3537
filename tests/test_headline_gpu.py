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


def _bwd(c, x, g, k=2, mfma=False):
    from spear_amd import _btp

    B, H, _, L = x.shape
    dx = torch.empty_like(x)
    dA = torch.empty(B, H, L, device=DEV, dtype=torch.float32)
    ck = torch.empty(B, H, L // 16, 16, device=DEV, dtype=torch.float32)
    _btp.backward(c, x, g, ck, dx, dA, k, 32, flags=_btp.FLAG_PATH_MFMA if mfma else 0)
    return dx, dA


CONFIGS = {
    "c3_B1024_H32_L128": dict(B=1024, H=32, L=128, seed=1234, x_std=0.25, gate="sigmoid"),
    "c4_B16_H64_L8192": dict(B=16, H=64, L=8192, seed=1235, x_std=0.25, gate="sigmoid"),
    "c5_B64_H128_L2048": dict(B=64, H=128, L=2048, seed=1236, x_std=1.0, gate="mixed"),
    # not a benchmark shape: rows of 4064 bytes, which do not end on a 128-byte line. Forward and backward move whole
    # lines there (their wavefronts pass row ends to each other through LDS); the fp32-dx check mode keeps the plain
    # movement, so the bit-equality checks of dx and dA below compare the two.
    "rows_off_lines_B64_H128_L2032": dict(B=64, H=128, L=2032, seed=1237, x_std=0.25, gate="sigmoid"),
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
    dxm, dAm = _bwd(c, xx, g, mfma=True)  # the matrix-core backward at full size
    torch.cuda.synchronize()
    assert torch.isfinite(y32).all() and torch.isfinite(dx.float()).all() and torch.isfinite(dA).all()
    assert torch.isfinite(dxm.float()).all() and torch.isfinite(dAm).all()

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
        # decay operands in two 16-bit pieces: 2^-15 of the sum of the terms' magnitudes (the oracle on |x|, |dy|)
        assert_close(f64(dxm[b : b + 1, h : h + 1]), rdx, BF16_ATOL, BF16_RTOL, f"dx mfma[{b},{h}]")
        magnitude = orc.backward(a_, np.abs(x_), np.abs(g_))[1]
        err = np.abs(f64(dAm[b : b + 1, h : h + 1]) - rdA)
        assert (err <= 1e-4 + 2.0 ** -15 * magnitude).all(), f"dA mfma[{b},{h}]: {err.max():.3e}"


@pytest.mark.parametrize("name", list(CONFIGS))
def test_every_row_of_the_benchmark_shapes_against_the_oracle(name):
    """Every (batch, head) row of B1024·H32·L128 (32,768 rows), B16·H64·L8192 (1,024), B64·H128·L2048 (8,192) and of
    B64·H128·L2032 (rows that do not end on a cache line), not a sample: fp32 `y`, unrounded `dx` (check mode) and `dA` within 1e-4, bf16 `y` and `dx` within 2e-2 of the float64
    oracle run on the same bf16-rounded inputs (the protocol of spear/ops/btp/runners.py:103-164), the oracle called
    on about half a million (token, head) units at a time."""
    from spear_amd import _btp

    cfg = CONFIGS[name]
    B, H, L = cfg["B"], cfg["H"], cfg["L"]
    print(f"{name} all rows: generating inputs", flush=True)
    coeff, x, dy = make_inputs(B, H, L, cfg["seed"], x_std=cfg["x_std"], gate=cfg["gate"])
    c, xx, g = coeff.to(DEV), x.to(DEV), dy.to(DEV)
    y32 = _fwd(c, xx, out_dtype=torch.float32)
    y16 = _fwd(c, xx)
    dx16, dA = _bwd(c, xx, g)
    dx32 = torch.empty(B, H, 16, L, device=DEV, dtype=torch.float32)
    dA_check = torch.empty(B, H, L, device=DEV, dtype=torch.float32)
    ck = torch.empty(0, device=DEV, dtype=torch.float32)
    _btp.backward(c, xx, g, ck, dx32, dA_check, 2, 32, flags=_btp.FLAG_DX_F32)
    torch.cuda.synchronize()
    assert torch.equal(dA_check, dA) and torch.equal(dx32.to(torch.bfloat16), dx16)
    got = {n: t.cpu() for n, t in (("y32", y32), ("y16", y16), ("dx16", dx16), ("dx32", dx32), ("dA", dA))}
    del y32, y16, dx16, dx32, dA, dA_check, c, xx, g
    torch.cuda.empty_cache()
    # rows are independent: the oracle sees the tensors as [B*H, 1, ...] and takes a slice of rows at a time
    rows = B * H
    flat = {n: t.reshape(rows, 1, *t.shape[2:]) for n, t in got.items()}
    cf, xf, gf = coeff.reshape(rows, 1, L), x.reshape(rows, 1, 16, L), dy.reshape(rows, 1, 16, L)
    worst = {n: 0.0 for n in got}
    step = max(1, (1 << 19) // L)
    for r0 in range(0, rows, step):
        if (r0 // step) % 8 == 0:
            print(f"{name} all rows: oracle on rows {r0}.. of {rows}", flush=True)
        sl = slice(r0, r0 + step)
        a_, x_, g_ = f64(cf[sl]), f64(xf[sl]), f64(gf[sl])
        ry = orc.forward(a_, x_)
        rdx, rdA = orc.backward(a_, x_, g_)
        for n, ref, atol, rtol in (("y32", ry, F32_ATOL, F32_RTOL), ("y16", ry, BF16_ATOL, BF16_RTOL),
                                   ("dx32", rdx, F32_ATOL, F32_RTOL), ("dx16", rdx, BF16_ATOL, BF16_RTOL),
                                   ("dA", rdA, F32_ATOL, F32_RTOL)):
            part = f64(flat[n][sl])
            assert_close(part, ref, atol, rtol, f"{n}[rows {r0}:{r0 + step}]")
            worst[n] = max(worst[n], float(np.abs(part - ref).max()))
    print(f"{name} all rows: max |err| " + ", ".join(f"{k} {v:.2e}" for k, v in worst.items()), flush=True)


def _free_gib():
    free, _ = torch.cuda.mem_get_info()
    return free / 2**30


def test_rows_past_2_31_elements_equal_the_same_rows_run_alone():
    """64-bit addressing: tensors of more than 2^31 elements (4.6 GB each in bf16). Every (b, h) row is
    independent, so the rows that lie beyond the 2^31-element mark must come out bit-identical to a
    call on those rows alone (offsets near zero)."""
    if _free_gib() < 48:
        pytest.skip("needs about 40 GiB of device memory")
    rows, L = 1100, 131072                      # 1100 * 16 * 131072 = 2.31e9 elements
    assert rows * 16 * L > 2**31
    g = torch.Generator(device=DEV).manual_seed(77)
    print("scan kernels past 2^31: inputs", flush=True)
    coeff = torch.sigmoid(torch.randn(1, rows, L, device=DEV, generator=g)).bfloat16()
    x = torch.empty(1, rows, 16, L, device=DEV, dtype=torch.bfloat16).normal_(0, 0.25, generator=g)
    dy = torch.empty(1, rows, 16, L, device=DEV, dtype=torch.bfloat16).normal_(0, 1, generator=g)
    print("scan kernels past 2^31: forward/backward", flush=True)
    y = _fwd(coeff, x)
    dx, dA = _bwd(coeff, x, dy)
    torch.cuda.synchronize()
    for lo, hi in ((0, 2), (1023, 1026), (rows - 3, rows)):   # row 1024 starts exactly at element 2^31
        sub = slice(lo, hi)
        cs, xs, gs = (t[:, sub].contiguous() for t in (coeff, x, dy))
        assert torch.equal(_fwd(cs, xs), y[:, sub]), f"y rows {lo}:{hi}"
        dxs, dAs = _bwd(cs, xs, gs)
        assert torch.equal(dxs, dx[:, sub]), f"dx rows {lo}:{hi}"
        assert torch.equal(dAs, dA[:, sub]), f"dA rows {lo}:{hi}"
    # and against the oracle on the head of the last row (a block depends on itself and its predecessor only)
    n = 256
    a_, x_ = f64(coeff[:, -1:, :n].cpu()), f64(x[:, -1:, :, :n].cpu())
    assert_close(f64(y[:, -1:, :, :n].cpu()), orc.forward(a_, x_), BF16_ATOL, BF16_RTOL, "y last row")


def test_fused_and_prefill_batches_past_2_31_elements_equal_the_same_batch_run_alone():
    from spear_amd import _btp

    if _free_gib() < 64:
        pytest.skip("needs about 50 GiB of device memory")
    g = torch.Generator(device=DEV).manual_seed(78)
    B, L, H = 5, 1 << 20, 32                    # 5 * 2^20 * 512 = 2.68e9 elements; batch row 4 starts at 2^31
    F = H * 16
    print("fused kernels past 2^31: inputs", flush=True)
    a = torch.empty(B, L, H, device=DEV, dtype=torch.bfloat16).normal_(0, 1, generator=g)
    b, c, v, dout = (torch.empty(B, L, F, device=DEV, dtype=torch.bfloat16).normal_(0, 1, generator=g) for _ in range(4))
    out = torch.empty_like(v)
    grads = [torch.empty_like(t) for t in (a, b, c, v)]
    print("fused kernels past 2^31: forward/backward", flush=True)
    _btp.mix_forward(a, b, c, v, out, H, H)
    _btp.mix_backward(a, b, c, v, dout, *grads, H, H)
    torch.cuda.synchronize()
    last = [t[B - 1:].contiguous() for t in (a, b, c, v, dout)]
    out1 = torch.empty_like(last[3])
    grads1 = [torch.empty_like(t) for t in last[:4]]
    _btp.mix_forward(*last[:4], out1, H, H)
    _btp.mix_backward(*last, *grads1, H, H)
    torch.cuda.synchronize()
    assert torch.equal(out1, out[B - 1:])
    for name, g1, gall in zip("abcv", grads1, grads):
        assert torch.equal(g1, gall[B - 1:]), f"d{name}"
    del a, b, c, v, dout, out, grads, last, out1, grads1
    torch.cuda.empty_cache()

    rows, Lp = 1100, 131072
    print("prefill past 2^31: inputs", flush=True)
    A = torch.sigmoid(torch.randn(1, rows, Lp, device=DEV, generator=g)).bfloat16()
    X, C, V = (torch.empty(1, rows, 16, Lp, device=DEV, dtype=torch.bfloat16).normal_(0, 0.5, generator=g) for _ in range(3))

    def prefill(A_, X_, C_, V_):
        n = A_.shape[1]
        Y = torch.empty_like(X_)
        h, cp = (torch.empty(1, n, 16, device=DEV) for _ in range(2))
        r = torch.empty(1, n, device=DEV)
        _btp.jagged_prefill(A_, X_, C_, V_, None, Y, h, r, cp, 16, False)
        return Y, h, r, cp

    print("prefill past 2^31: run", flush=True)
    whole = prefill(A, X, C, V)
    sub = slice(rows - 3, rows)
    part = prefill(*(t[:, sub].contiguous() for t in (A, X, C, V)))
    torch.cuda.synchronize()
    for name, w, p in zip(("Y", "h", "r", "c_prev"), whole, part):
        assert torch.equal(p, w[:, sub]), name
