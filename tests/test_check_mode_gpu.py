"""The fp32 check mode: every output and every gradient of the kernels as the kernels' own fp32 values
(no final rounding to 16 bits), held to the north-star bound for that mode, 1e-4 absolute + relative
against the float64 oracle on the same 16-bit inputs.

  stand-alone op     y  (fp32 output dtype), dA (always fp32), dx with SPEAR_BTP_DX_F32
  log-gate op        the same with fp32 gates, dgate
  fused / q k v gate out, dq, dk, dv, dgate (da, db, dc, dv) with SPEAR_MIX_F32_RESULTS

The 16-bit results of the default mode must be exactly the rounding of these."""

import numpy as np
import pytest
import torch

from helpers import F32_ATOL, F32_RTOL, assert_close, f64, make_inputs
from oracle import btp_oracle as orc
from test_btp_gpu import SHAPES, _sweep_cases
from test_headline_gpu import CONFIGS

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def backward_f32(coeff, x, dy, k=2):
    """dx (fp32, unrounded), dx (x.dtype) and dA of the stand-alone backward, device tensors in and out."""
    from spear_amd import _btp

    B, H, _, L = x.shape
    ck = torch.empty((B, H, L // 16, 16), device=DEV, dtype=torch.float32)
    dx32 = torch.full((B, H, 16, L), float("nan"), device=DEV, dtype=torch.float32)
    dA32 = torch.full((B, H, L), float("nan"), device=DEV, dtype=torch.float32)
    _btp.backward(coeff, x, dy, ck, dx32, dA32, k, 32, flags=_btp.FLAG_DX_F32)
    dx16 = torch.full((B, H, 16, L), float("nan"), device=DEV, dtype=x.dtype)
    dA = torch.full((B, H, L), float("nan"), device=DEV, dtype=torch.float32)
    _btp.backward(coeff, x, dy, ck, dx16, dA, k, 32)
    torch.cuda.synchronize()
    assert torch.equal(dA, dA32), "dA must not depend on the dx mode"
    return dx32, dx16, dA


@pytest.mark.parametrize("k", [2, 1])
@pytest.mark.parametrize("B,H,L", SHAPES)
def test_dx_fp32_matches_oracle_to_1e4(B, H, L, k):
    coeff, x, dy = make_inputs(B, H, L, seed=1300 + L + k)
    print(f"dx f32 B={B} H={H} L={L} k={k}", flush=True)
    dx32, dx16, dA = backward_f32(coeff.to(DEV), x.to(DEV), dy.to(DEV), k)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy), k=k)
    assert_close(f64(dx32), rdx, F32_ATOL, F32_RTOL, "dx fp32")
    assert_close(f64(dA), rdA, F32_ATOL, F32_RTOL, "dA")
    assert torch.equal(dx16, dx32.to(x.dtype)), "the 16-bit dx must be the rounding of the fp32 dx"


@pytest.mark.parametrize("B,H,L,k,f32,seed", _sweep_cases())
def test_dx_fp32_on_odd_launch_shapes(B, H, L, k, f32, seed):
    """Ragged spans, partial workgroups, hand-over and halo edges (the sweep of test_btp_gpu), dx unrounded."""
    coeff, x, dy = make_inputs(B, H, L, seed=seed, stress=1.5)
    if f32:
        dy = dy.float()
    print(f"dx f32 sweep B={B} H={H} L={L} k={k} f32dy={f32} seed={seed}", flush=True)
    dx32, dx16, dA = backward_f32(coeff.to(DEV), x.to(DEV), dy.to(DEV), k)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy), k=k)
    assert_close(f64(dx32), rdx, F32_ATOL, F32_RTOL, "dx fp32")
    assert_close(f64(dA), rdA, F32_ATOL, F32_RTOL, "dA")
    assert torch.equal(dx16, dx32.to(x.dtype))


def test_dx_fp32_fp16_inputs_and_log_gates():
    from spear_amd import _btp

    coeff, x, dy = make_inputs(2, 3, 400, seed=1401, dtype=torch.float16)
    dx32, dx16, dA = backward_f32(coeff.to(DEV), x.to(DEV), dy.to(DEV))
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy))
    assert_close(f64(dx32), rdx, F32_ATOL, F32_RTOL, "dx fp32 (fp16 inputs)")
    assert torch.equal(dx16, dx32.half())

    # fp32 log-space gates: a = exp(gate) is formed in fp32 inside the kernel, the oracle sees exp in float64
    g = torch.Generator().manual_seed(1402)
    gate = -torch.nn.functional.softplus(torch.randn(2, 4, 272, generator=g))
    gate[1, 2] = -1e-4 * torch.rand(272, generator=g)  # near-identity head
    _, x, dy = make_inputs(2, 4, 272, seed=1403)
    dx32 = torch.full((2, 4, 16, 272), float("nan"), device=DEV)
    dgate = torch.full((2, 4, 272), float("nan"), device=DEV)
    _btp.backward_log(gate.to(DEV), x.to(DEV), dy.to(DEV), dx32, dgate, 2)
    dx16 = torch.empty(2, 4, 16, 272, device=DEV, dtype=torch.bfloat16)
    _btp.backward_log(gate.to(DEV), x.to(DEV), dy.to(DEV), dx16, torch.empty_like(dgate), 2)
    torch.cuda.synchronize()
    a = np.exp(f64(gate))
    rdx, rdA = orc.backward(a, f64(x), f64(dy))
    assert_close(f64(dx32), rdx, F32_ATOL, F32_RTOL, "dx fp32 (log gates)")
    assert_close(f64(dgate), rdA * a, F32_ATOL, F32_RTOL, "dgate")
    assert torch.equal(dx16, dx32.bfloat16())


@pytest.mark.parametrize("name", list(CONFIGS))
def test_dx_fp32_on_sampled_rows_of_the_benchmark_shapes(name):
    cfg = CONFIGS[name]
    B, H, L = cfg["B"], cfg["H"], cfg["L"]
    print(f"{name}: generating inputs", flush=True)
    coeff, x, dy = make_inputs(B, H, L, cfg["seed"], x_std=cfg["x_std"], gate=cfg["gate"])
    dx32, dx16, dA = backward_f32(coeff.to(DEV), x.to(DEV), dy.to(DEV))
    assert torch.equal(dx16, dx32.bfloat16())
    print(f"{name}: oracle on sampled rows", flush=True)
    rng = np.random.default_rng(cfg["seed"] + 1)
    for b, h in zip(rng.integers(0, B, size=8), rng.integers(0, H, size=8)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        rdx, rdA = orc.backward(f64(coeff[sl]), f64(x[sl]), f64(dy[sl]))
        assert_close(f64(dx32[sl]), rdx, F32_ATOL, F32_RTOL, f"dx fp32 [{b},{h}]")
        assert_close(f64(dA[sl]), rdA, F32_ATOL, F32_RTOL, f"dA [{b},{h}]")


# ---- fused kernels --------------------------------------------------------------------------------
def _mix_inputs(B, L, H, Hkv, seed, qkv, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    if qkv:
        a = -torch.nn.functional.softplus(torch.randn(B, L, H, generator=g))
    else:
        a = (torch.randn(B, L, H, generator=g) * scale).bfloat16()
    b = (torch.randn(B, L, Hkv * 16, generator=g) * (0.25 if qkv else scale)).bfloat16()
    c = (torch.randn(B, L, Hkv * 16, generator=g) * (0.25 if qkv else 1.0)).bfloat16()
    v = (torch.randn(B, L, H * 16, generator=g) * (0.25 if qkv else 1.0)).bfloat16()
    dout = torch.randn(B, L, H * 16, generator=g).bfloat16()
    return a, b, c, v, dout


def _mix_run(ins, H, Hkv, qkv, f32):
    from spear_amd import _btp

    a, b, c, v, dout = (t.to(DEV) for t in ins)
    rt = torch.float32 if f32 else v.dtype
    out = torch.full(v.shape, float("nan"), device=DEV, dtype=rt)
    _btp.mix_forward(a, b, c, v, out, H, Hkv, qkv_gate=qkv)
    grads = [torch.full(t.shape, float("nan"), device=DEV, dtype=torch.float32 if (f32 or t.dtype == torch.float32) else t.dtype)
             for t in (a, b, c, v)]
    _btp.mix_backward(a, b, c, v, dout, *grads, H, Hkv, qkv_gate=qkv)
    torch.cuda.synchronize()
    return out, grads


def _mix_oracle(ins, H, Hkv, qkv):
    a, b, c, v, dout = (f64(t) for t in ins)
    if qkv:  # b is k, c is q, a is the log-decay gate; gradients come back in operand order (a, b, c, v)
        return orc.qkv_gate_forward(c, b, v, a, H, Hkv), list(orc.qkv_gate_backward(c, b, v, a, dout, H, Hkv))
    return orc.phalanx_mix_forward(a, b, c, v, H, Hkv), list(orc.phalanx_mix_backward(a, b, c, v, dout, H, Hkv))


# head groupings summed inside a wavefront (1, 2, 4, 8 heads per kv head) and through LDS (3, 6, 12, 16), odd head counts
@pytest.mark.parametrize("qkv", [False, True], ids=["layer", "qkv_gate"])
@pytest.mark.parametrize("B,L,H,Hkv", [(1, 16, 4, 4), (2, 48, 8, 8), (3, 128, 8, 2), (2, 144, 16, 4), (1, 512, 32, 32),
                                       (2, 272, 12, 3), (1, 1040, 4, 1), (1, 4096, 8, 8), (2, 2064, 16, 2),
                                       (2, 80, 6, 2), (1, 144, 12, 2), (2, 64, 12, 1), (1, 272, 16, 1), (2, 48, 5, 5),
                                       (1, 96, 3, 1)])
def test_fused_results_fp32_match_oracle_to_1e4(B, L, H, Hkv, qkv):
    ins = _mix_inputs(B, L, H, Hkv, seed=1500 + L + H, qkv=qkv)
    print(f"fused f32 B={B} L={L} H={H} Hkv={Hkv} qkv={qkv}", flush=True)
    out32, g32 = _mix_run(ins, H, Hkv, qkv, f32=True)
    out16, g16 = _mix_run(ins, H, Hkv, qkv, f32=False)
    ref_out, ref_g = _mix_oracle(ins, H, Hkv, qkv)
    # the layer form evaluates two sigmoids with the hardware's exp and reciprocal (relative error ~1e-6
    # each), which the 1e-4 bound covers
    assert_close(f64(out32), ref_out, F32_ATOL, F32_RTOL, "out fp32")
    for name, got, ref in zip(("da/dgate", "db/dk", "dc/dq", "dv"), g32, ref_g):
        assert_close(f64(got), ref, F32_ATOL, F32_RTOL, name + " fp32")
    assert torch.equal(out16, out32.to(out16.dtype))
    for name, lo, hi in zip(("da/dgate", "db/dk", "dc/dq", "dv"), g16, g32):
        assert torch.equal(lo, hi.to(lo.dtype)), name


@pytest.mark.parametrize("qkv", [False, True], ids=["layer", "qkv_gate"])
@pytest.mark.parametrize("B,L,H,Hkv", [(2, 48, 8, 8), (3, 128, 8, 2), (2, 272, 12, 3), (16, 256, 16, 16)])
def test_fused_fp16_results_are_the_rounded_fp32_results(B, L, H, Hkv, qkv):
    """fp16 tensors through the fused kernels: every 16-bit result is the fp32 result of the check mode rounded to
    nearest even (the conversion is not folded into the arithmetic before it, where a single rounding from the exact
    sum would differ at ties)."""
    ins = _mix_inputs(B, L, H, Hkv, seed=1700 + L + H, qkv=qkv)
    ins = tuple(t.half() if t.dtype == torch.bfloat16 else t for t in ins)
    print(f"fused fp16 B={B} L={L} H={H} Hkv={Hkv} qkv={qkv}", flush=True)
    out32, g32 = _mix_run(ins, H, Hkv, qkv, f32=True)
    out16, g16 = _mix_run(ins, H, Hkv, qkv, f32=False)
    assert out16.dtype == torch.float16
    assert torch.equal(out16, out32.to(out16.dtype))
    for name, lo, hi in zip(("da/dgate", "db/dk", "dc/dq", "dv"), g16, g32):
        assert torch.equal(lo, hi.to(lo.dtype)), name
    ref_out, ref_g = _mix_oracle(ins, H, Hkv, qkv)
    assert_close(f64(out32), ref_out, F32_ATOL, F32_RTOL, "out fp32")
