"""Parity of the HIP kernels (called through the C ABI via spear_amd._btp) with the CPU oracle.

Tolerances are the north-star ones: bf16 I/O within 2e-2 (absolute + relative), fp32 outputs of
the exact-fp32 path within 1e-4, both against the float64 oracle evaluated on the same
bf16-rounded inputs."""

import numpy as np
import pytest
import torch

from helpers import BF16_ATOL, BF16_RTOL, F32_ATOL, F32_RTOL, assert_close, f64, make_inputs
from oracle import btp_oracle as orc

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def run_forward(coeff, x, k=2, out_dtype=torch.bfloat16, checkpoint=False, mfma=False):
    from spear_amd import _btp

    c, xx = coeff.to(DEV), x.to(DEV)
    B, H, _, L = x.shape
    y = torch.full((B, H, 16, L), float("nan"), device=DEV, dtype=out_dtype)
    ck = torch.full((B, H, L // 16, 16), float("nan"), device=DEV, dtype=torch.float32)
    flags = (_btp.FLAG_WRITE_CHECKPOINT if checkpoint else 0) | (_btp.FLAG_PATH_MFMA if mfma else 0)
    _btp.forward(c, xx, y, ck, k, 32, flags=flags)
    torch.cuda.synchronize()
    return (y.cpu(), ck.cpu()) if checkpoint else y.cpu()


def run_backward(coeff, x, dy, k=2, mfma=False):
    from spear_amd import _btp

    c, xx, g = coeff.to(DEV), x.to(DEV), dy.to(DEV)
    B, H, _, L = x.shape
    dx = torch.full((B, H, 16, L), float("nan"), device=DEV, dtype=x.dtype)
    dA = torch.full((B, H, L), float("nan"), device=DEV, dtype=torch.float32)
    ck = torch.empty((B, H, L // 16, 16), device=DEV, dtype=torch.float32)
    _btp.backward(c, xx, g, ck, dx, dA, k, 32, flags=_btp.FLAG_PATH_MFMA if mfma else 0)
    torch.cuda.synchronize()
    return dx.cpu(), dA.cpu()


SHAPES = [(1, 1, 16), (2, 3, 32), (1, 2, 48), (2, 2, 64), (1, 2, 128), (2, 2, 144), (1, 3, 256), (2, 8, 512), (1, 2, 1040), (3, 5, 112)]


@pytest.mark.parametrize("k", [2, 1])
@pytest.mark.parametrize("B,H,L", SHAPES)
def test_forward_bf16_matches_oracle(B, H, L, k):
    coeff, x, _ = make_inputs(B, H, L, seed=100 + L + k)
    print(f"fwd bf16 B={B} H={H} L={L} k={k}", flush=True)
    y = run_forward(coeff, x, k=k)
    assert_close(f64(y), orc.forward(f64(coeff), f64(x), k=k), BF16_ATOL, BF16_RTOL, "y")


@pytest.mark.parametrize("k", [2, 1])
@pytest.mark.parametrize("B,H,L", SHAPES)
def test_forward_fp32_out_matches_oracle_to_1e4(B, H, L, k):
    coeff, x, _ = make_inputs(B, H, L, seed=200 + L + k)
    print(f"fwd f32 B={B} H={H} L={L} k={k}", flush=True)
    y = run_forward(coeff, x, k=k, out_dtype=torch.float32)
    assert_close(f64(y), orc.forward(f64(coeff), f64(x), k=k), F32_ATOL, F32_RTOL, "y")


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("k", [2, 1])
@pytest.mark.parametrize("B,H,L", SHAPES)
def test_forward_mfma_path_matches_oracle(B, H, L, k, out_dtype):
    # the MFMA path feeds its decay matrix to the matrix cores as two 16-bit pieces (hi + lo), so its fp32 output
    # is held to the fp32 bound like the recurrence kernel's (the reference rounds the matrix to bf16 once)
    coeff, x, _ = make_inputs(B, H, L, seed=700 + L + k)
    print(f"fwd mfma B={B} H={H} L={L} k={k} {out_dtype}", flush=True)
    y = run_forward(coeff, x, k=k, out_dtype=out_dtype, mfma=True)
    atol, rtol = (F32_ATOL, F32_RTOL) if out_dtype == torch.float32 else (BF16_ATOL, BF16_RTOL)
    assert_close(f64(y), orc.forward(f64(coeff), f64(x), k=k), atol, rtol, "y")


@pytest.mark.parametrize("B,H,L,k", [(2, 3, 64, 2), (1, 2, 400, 2), (2, 2, 144, 1)])
def test_forward_mfma_path_fp16(B, H, L, k):
    coeff, x, _ = make_inputs(B, H, L, seed=900 + L, dtype=torch.float16)
    y = run_forward(coeff, x, k=k, out_dtype=torch.float16, mfma=True)
    # fp16 storage (11 significant bits) of the decay matrix and of y
    assert_close(f64(y), orc.forward(f64(coeff), f64(x), k=k), 4e-3, 4e-3, "y mfma fp16")
    y32 = run_forward(coeff, x, k=k, out_dtype=torch.float32, mfma=True)
    assert_close(f64(y32), orc.forward(f64(coeff), f64(x), k=k), F32_ATOL, F32_RTOL, "y32 mfma fp16")


def test_forward_mfma_path_stress_and_zero_coefficients():
    coeff, x, _ = make_inputs(2, 8, 2048, seed=1236, gate="mixed")
    y = run_forward(coeff, x, mfma=True)
    assert_close(f64(y), orc.forward(f64(coeff), f64(x)), BF16_ATOL, BF16_RTOL, "y mixed gates")
    coeff, x, _ = make_inputs(1, 2, 160, seed=7)
    coeff[0, 0, [0, 5, 16, 33, 127, 128]] = 0.0
    y = run_forward(coeff, x, out_dtype=torch.float32, mfma=True)
    assert_close(f64(y), orc.forward(f64(coeff), f64(x)), F32_ATOL, F32_RTOL, "y zero coefficients")


def test_mfma_path_rejects_what_it_does_not_do():
    from spear_amd import _btp

    coeff, x, dy = make_inputs(1, 2, 32, seed=1)
    c, xx = coeff.to(DEV), x.to(DEV)
    y = torch.empty_like(xx)
    ck = torch.empty(1, 2, 2, 16, device=DEV)
    with pytest.raises(RuntimeError, match="does not store the carry checkpoint"):
        _btp.forward(c, xx, y, ck, 2, 32, flags=_btp.FLAG_PATH_MFMA | _btp.FLAG_WRITE_CHECKPOINT)
    dA = torch.empty(1, 2, 32, device=DEV)
    with pytest.raises(RuntimeError, match="no fp32 dx"):
        _btp.backward(c, xx, dy.to(DEV), ck, torch.empty_like(xx, dtype=torch.float32), dA, 2, 32,
                      flags=_btp.FLAG_PATH_MFMA | _btp.FLAG_DX_F32)
    # an fp32 dy (the reference accepts one, csrc/btp/_bindings.cu:52-59, and rounds it for its MMA) is refused, not
    # rounded behind the caller's back
    with pytest.raises(RuntimeError, match="takes dy in the inputs' 16-bit type"):
        _btp.backward(c, xx, dy.to(DEV).float(), ck, torch.empty_like(xx), dA, 2, 32, flags=_btp.FLAG_PATH_MFMA)


# The matrix-core backward takes its decay operands as two 16-bit pieces (hi + lo: about 2^-17 per entry with bf16).
# dA_r is a sum over channels and (source, sink) pairs of products decay * x * dy in which two rounded decay entries
# meet, so its error is at most about 2 * 2^-17 of the sum of the terms' magnitudes -- which the oracle gives exactly
# when it is run on |x| and |dy| (the decays are not negative). `eps` is that factor.
def assert_dA_from_rounded_decays(dA, coeff, x, dy, k, what, eps=2.0 ** -15):
    rdA = orc.backward(f64(coeff), f64(x), f64(dy), k=k)[1]
    magnitude = orc.backward(f64(coeff), np.abs(f64(x)), np.abs(f64(dy)), k=k)[1]
    err = np.abs(f64(dA) - rdA)
    bound = 1e-4 + eps * magnitude
    worst = np.argmax(err - bound)
    assert (err <= bound).all(), f"{what}: max |err|={err.max():.3e}; worst at {worst}: err {err.flat[worst]:.3e} bound {bound.flat[worst]:.3e}"
    # and the bound is not vacuous: it stays a small fraction of the gradient's own scale
    assert np.median(bound) < 0.05 * max(np.abs(rdA).max(), 1.0), what


@pytest.mark.parametrize("k", [2, 1])
@pytest.mark.parametrize("B,H,L", SHAPES)
def test_backward_mfma_path_matches_oracle(B, H, L, k):
    coeff, x, dy = make_inputs(B, H, L, seed=350 + L + k)
    print(f"bwd mfma B={B} H={H} L={L} k={k}", flush=True)
    dx, dA = run_backward(coeff, x, dy, k=k, mfma=True)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy), k=k)
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx mfma")
    assert_dA_from_rounded_decays(dA, coeff, x, dy, k, "dA mfma")


def test_backward_mfma_path_fp16_stress_and_zero_coefficients():
    coeff, x, dy = make_inputs(2, 3, 272, seed=351, dtype=torch.float16)
    dx, dA = run_backward(coeff, x, dy, mfma=True)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy))
    assert_close(f64(dx), rdx, 4e-3, 4e-3, "dx mfma fp16")
    assert_dA_from_rounded_decays(dA, coeff, x, dy, 2, "dA mfma fp16")
    coeff, x, dy = make_inputs(2, 8, 2048, seed=1236, gate="mixed")
    dx, dA = run_backward(coeff, x, dy, mfma=True)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy))
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx mixed gates")
    assert_dA_from_rounded_decays(dA, coeff, x, dy, 2, "dA mixed gates")
    coeff, x, dy = make_inputs(1, 2, 160, seed=7)
    coeff[0, 0, [0, 5, 16, 33, 127, 128]] = 0.0
    dx, dA = run_backward(coeff, x, dy, mfma=True)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy))
    assert torch.isfinite(dx.float()).all() and torch.isfinite(dA).all()
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx zero coefficients")
    assert_dA_from_rounded_decays(dA, coeff, x, dy, 2, "dA zero coefficients")


@pytest.mark.parametrize("k", [2, 1])
@pytest.mark.parametrize("B,H,L", SHAPES)
def test_backward_bf16_matches_oracle(B, H, L, k):
    coeff, x, dy = make_inputs(B, H, L, seed=300 + L + k)
    print(f"bwd bf16 B={B} H={H} L={L} k={k}", flush=True)
    dx, dA = run_backward(coeff, x, dy, k=k)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy), k=k)
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx")
    # dA is an fp32 output computed in fp32 from exact inputs: hold it to the fp32 bound
    assert_close(f64(dA), rdA, F32_ATOL, F32_RTOL, "dA")


@pytest.mark.parametrize("B,H,L", [(2, 3, 32), (2, 2, 144), (2, 8, 512)])
def test_backward_fp32_dy(B, H, L):
    coeff, x, _ = make_inputs(B, H, L, seed=400 + L)
    dy = torch.randn(B, H, 16, L, generator=torch.Generator().manual_seed(L))
    print(f"bwd f32-dy B={B} H={H} L={L}", flush=True)
    dx, dA = run_backward(coeff, x, dy)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy))
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx")
    assert_close(f64(dA), rdA, F32_ATOL, F32_RTOL, "dA")


@pytest.mark.parametrize("B,H,L", [(2, 3, 64), (1, 2, 400), (4, 25, 48), (3, 7, 2032), (64, 8, 128)])
def test_fp16_inputs(B, H, L):
    """fp16 tensors against the oracle, and the fp16 results are the fp32 results (fp32 y, check-mode dx) rounded to
    nearest even: the conversion is not folded into the arithmetic before it, where one rounding from the exact sum
    would differ at ties, in some kernel instances and not in others (the carry store picks another instance)."""
    from spear_amd import _btp

    coeff, x, dy = make_inputs(B, H, L, seed=500 + L, dtype=torch.float16)
    print(f"fp16 B={B} H={H} L={L}", flush=True)
    y = run_forward(coeff, x, out_dtype=torch.float16)
    assert_close(f64(y), orc.forward(f64(coeff), f64(x)), 2e-3, 2e-3, "y fp16")
    dx, dA = run_backward(coeff, x, dy)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy))
    assert_close(f64(dx), rdx, 2e-3, 2e-3, "dx fp16")
    assert_close(f64(dA), rdA, F32_ATOL, F32_RTOL, "dA")
    assert torch.equal(y, run_forward(coeff, x, out_dtype=torch.float32).to(torch.float16))
    assert torch.equal(y, run_forward(coeff, x, out_dtype=torch.float16, checkpoint=True)[0])
    c, xx, g = coeff.to(DEV), x.to(DEV), dy.to(DEV)
    dx32, dA32 = torch.empty(B, H, 16, L, device=DEV), torch.empty(B, H, L, device=DEV)
    _btp.backward(c, xx, g, torch.empty(0, device=DEV), dx32, dA32, 2, 32, flags=_btp.FLAG_DX_F32)
    assert torch.equal(dx, dx32.to(torch.float16).cpu()) and torch.equal(dA, dA32.cpu())


@pytest.mark.parametrize("L", [64, 272])
def test_checkpoint_matches_oracle(L):
    coeff, x, _ = make_inputs(2, 3, L, seed=600 + L)
    print(f"checkpoint L={L}", flush=True)
    y, ck = run_forward(coeff, x, checkpoint=True)
    ry, rck = orc.forward(f64(coeff), f64(x), with_checkpoint=True)
    assert_close(f64(y), ry, BF16_ATOL, BF16_RTOL, "y")
    nb = L // 16
    assert_close(f64(ck)[:, :, : nb - 1], rck[:, :, : nb - 1], F32_ATOL, F32_RTOL, "checkpoint")
    assert torch.isnan(ck[:, :, nb - 1]).all(), "the last checkpoint slot must stay untouched"


@pytest.mark.parametrize("stress", [2.5, 4.0])
def test_stressed_gates(stress):
    # sigmoid(N(0, stress)) coefficients as in the reference's stress sweeps (tests/btp/test_numerics.py:104-166)
    coeff, x, dy = make_inputs(2, 4, 512, seed=321, stress=stress)
    print(f"stress={stress}", flush=True)
    y = run_forward(coeff, x, out_dtype=torch.float32)
    assert_close(f64(y), orc.forward(f64(coeff), f64(x)), F32_ATOL, F32_RTOL, "y")
    dx, dA = run_backward(coeff, x, dy)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy))
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx")
    assert_close(f64(dA), rdA, F32_ATOL, F32_RTOL, "dA")


def test_log_space_stress_mixture():
    # per head either exp(U[-20,-5]) (near-total forgetting) or exp(U[-1e-4,0]) (near-identity)
    coeff, x, dy = make_inputs(2, 8, 2048, seed=1236, gate="mixed")
    print("mixed gates", flush=True)
    y = run_forward(coeff, x)
    assert_close(f64(y), orc.forward(f64(coeff), f64(x)), BF16_ATOL, BF16_RTOL, "y")
    dx, dA = run_backward(coeff, x, dy)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy))
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx")
    assert_close(f64(dA), rdA, F32_ATOL, F32_RTOL, "dA")


def test_zero_negative_and_tiny_coefficients():
    # at or below 1e-9 (and negative) counts as exactly zero, as in the reference kernels
    coeff, x, dy = make_inputs(1, 2, 160, seed=7)
    coeff[0, 0, [0, 5, 16, 33, 127, 128]] = 0.0
    coeff[0, 1, [3, 47, 48]] = -0.5
    coeff[0, 1, [100]] = 1e-12
    ref_coeff = f64(coeff).copy()
    ref_coeff[ref_coeff <= 1e-9] = 0.0
    print("zero coefficients", flush=True)
    y = run_forward(coeff, x, out_dtype=torch.float32)
    assert_close(f64(y), orc.forward(ref_coeff, f64(x)), F32_ATOL, F32_RTOL, "y")
    dx, dA = run_backward(coeff, x, dy)
    rdx, rdA = orc.backward(ref_coeff, f64(x), f64(dy))
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx")
    assert_close(f64(dA), rdA, F32_ATOL, F32_RTOL, "dA")


def test_outputs_are_deterministic():
    coeff, x, dy = make_inputs(2, 4, 256, seed=11)
    y1, y2 = run_forward(coeff, x), run_forward(coeff, x)
    assert torch.equal(y1, y2)
    (dx1, dA1), (dx2, dA2) = run_backward(coeff, x, dy), run_backward(coeff, x, dy)
    assert torch.equal(dx1, dx2) and torch.equal(dA1, dA2)


def test_empty_batch_is_a_noop():
    from spear_amd import _btp

    coeff = torch.empty(0, 4, 64, device=DEV, dtype=torch.bfloat16)
    x = torch.empty(0, 4, 16, 64, device=DEV, dtype=torch.bfloat16)
    y = torch.empty_like(x)
    ck = torch.empty(0, 4, 4, 16, device=DEV, dtype=torch.float32)
    _btp.forward(coeff, x, y, ck, 2, 32)
    torch.cuda.synchronize()


# ---- committed closed-form vectors (tests/golden) ------------------------------------------------
@pytest.mark.parametrize("k", [2, 1])
@pytest.mark.parametrize("case", ["smooth", "edges", "one_block"])
def test_kernels_match_committed_closed_form_vectors(case, k):
    from helpers import golden_vectors

    v = golden_vectors()[case]
    coeff, x, dy = (torch.from_numpy(v[n]).bfloat16() for n in ("coeff", "x", "dy"))
    for n, t in (("coeff", coeff), ("x", x), ("dy", dy)):
        assert np.array_equal(f64(t), v[n].astype(np.float64)), f"{n} is not bfloat16-exact"
    print(f"golden {case} k={k}", flush=True)
    assert_close(f64(run_forward(coeff, x, k=k)), v[f"k{k}.y"], BF16_ATOL, BF16_RTOL, "y bf16")
    assert_close(f64(run_forward(coeff, x, k=k, out_dtype=torch.float32)), v[f"k{k}.y"], F32_ATOL, F32_RTOL, "y fp32")
    dx, dA = run_backward(coeff, x, dy, k=k)
    assert_close(f64(dx), v[f"k{k}.dx"], BF16_ATOL, BF16_RTOL, "dx")
    assert_close(f64(dA), v[f"k{k}.dA"], BF16_ATOL, BF16_RTOL, "dA")
    assert_close(f64(run_forward(coeff, x, k=k, mfma=True)), v[f"k{k}.y"], BF16_ATOL, BF16_RTOL, "y mfma")
    dx, dA = run_backward(coeff, x, dy, k=k, mfma=True)
    assert_close(f64(dx), v[f"k{k}.dx"], BF16_ATOL, BF16_RTOL, "dx mfma")
    assert_close(f64(dA), v[f"k{k}.dA"], 2 * F32_ATOL, 2 * F32_RTOL, "dA mfma")


# ---- seeded sweep over odd launch shapes ---------------------------------------------------------
def _sweep_cases(n=36, seed=2024):
    rng = np.random.RandomState(seed)
    cases = []
    for i in range(n):
        B, H = int(rng.randint(1, 6)), int(rng.randint(1, 8))
        # lengths around span (128) and workgroup (4 or 8 spans) boundaries, plus ragged last spans
        L = 16 * int(rng.choice([1, 2, 7, 8, 9, 15, 16, 17, 24, 31, 32, 33, 40, 63, 64, 65, 72, 129]))
        if B * H * L > 60000:
            H = max(1, 60000 // (B * L))
        cases.append((B, H, L, int(rng.choice([1, 2, 2, 2])), bool(rng.randint(2)), 4000 + i))
    return cases


@pytest.mark.parametrize("B,H,L,k,f32,seed", _sweep_cases())
def test_forward_and_backward_on_odd_launch_shapes(B, H, L, k, f32, seed):
    """Rows that end inside a span, rows of 1..17 spans, span counts that do not fill the last workgroup:
    every hand-over / halo / early-exit combination of the launch geometry, against the oracle."""
    coeff, x, dy = make_inputs(B, H, L, seed=seed, stress=1.5)
    print(f"sweep B={B} H={H} L={L} k={k} f32={f32} seed={seed}", flush=True)
    out_dtype = torch.float32 if f32 else torch.bfloat16
    y = run_forward(coeff, x, k=k, out_dtype=out_dtype)
    atol, rtol = (F32_ATOL, F32_RTOL) if f32 else (BF16_ATOL, BF16_RTOL)
    assert_close(f64(y), orc.forward(f64(coeff), f64(x), k=k), atol, rtol, "y")
    if f32:
        dy = dy.float()
    c, xx, g = coeff.to(DEV), x.to(DEV), dy.to(DEV)
    from spear_amd import _btp

    dx = torch.full((B, H, 16, L), float("nan"), device=DEV, dtype=x.dtype)
    dA = torch.full((B, H, L), float("nan"), device=DEV, dtype=torch.float32)
    _btp.backward(c, xx, g, torch.empty((B, H, L // 16, 16), device=DEV), dx, dA, k, 32)
    rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy), k=k)
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx")
    assert_close(f64(dA), rdA, F32_ATOL, F32_RTOL, "dA")
    if not f32:  # the matrix-core backward on the same launch geometries (it takes dy in the inputs' type)
        dxm, dAm = run_backward(coeff, x, dy, k=k, mfma=True)
        assert_close(f64(dxm), rdx, BF16_ATOL, BF16_RTOL, "dx mfma")
        assert_dA_from_rounded_decays(dAm, coeff, x, dy, k, "dA mfma")


def _carve(shape, dtype, offset, fill):
    """A contiguous tensor of `shape` that starts `offset` elements into a larger buffer filled with `fill`."""
    n = int(np.prod(shape))
    buf = torch.full((n + offset + 64,), fill, device=DEV, dtype=dtype)
    return buf, buf[offset : offset + n].view(shape)


@pytest.mark.parametrize("offsets", [(0, 0, 0, 0), (8, 16, 24, 40), (56, 8, 0, 32)], ids=["on_lines", "offsets_a", "offsets_b"])
@pytest.mark.parametrize("B,H,L", [(2, 3, 144), (1, 2, 272), (3, 5, 400), (2, 2, 1040), (1, 3, 2032), (5, 1, 2000), (7, 3, 272)])
def test_rows_of_several_spans_that_do_not_end_on_a_cache_line(B, H, L, offsets):
    """Rows of several spans with L % 64 != 0 start at different offsets inside their 128-byte lines; where such rows
    fill their spans well (all lengths here but 144, which goes the way of the next test) forward and backward move
    whole lines and hand the ends of the rows from wavefront to wavefront (16-bit and fp32 y, 16-bit
    dy, linear and log-space gates; an fp32 dy and the fp32-dx check mode keep the plain movement). Tensors are placed at
    16-byte steps off the line grid (x, dy, y and dx each at their own), so every row start 0..7 chunks into a line
    occurs. Results against the oracle; the 16-bit results equal the rounded fp32 ones (y: another instance of the
    whole-line movement with rows twice as long; dx: the plain movement), the fp32-dy and log-gate instances agree
    with the 16-bit linear one, and nothing is written outside the tensors."""
    from spear_amd import _btp

    coeff, x, dy = make_inputs(B, H, L, seed=600 + L + offsets[0], stress=1.5)
    c = coeff.to(DEV)
    gate = torch.log(c.float())  # exp(gate) gives back the 16-bit decays to fp32 rounding
    shape = (B, H, 16, L)
    n = int(np.prod(shape))
    (bx, xv), (bg, gv) = _carve(shape, x.dtype, offsets[0], 0.0), _carve(shape, x.dtype, offsets[1], 0.0)
    bg32, gv32 = _carve(shape, torch.float32, offsets[1] // 2, 0.0)
    xv.copy_(x)
    gv.copy_(dy)
    gv32.copy_(dy)
    ck = torch.empty(0, device=DEV, dtype=torch.float32)

    def untouched(name, buf, off):
        assert bool((buf[:off] == 7).all()) and bool((buf[off + n :] == 7).all()), f"{name}: bytes outside the tensor changed"

    for k in (2, 1):
        print(f"rows off lines B={B} H={H} L={L} offsets={offsets} k={k}", flush=True)
        (by, yv), (bd, dxv) = _carve(shape, x.dtype, offsets[2], 7.0), _carve(shape, x.dtype, offsets[3], 7.0)
        by32, y32 = _carve(shape, torch.float32, offsets[2] // 2, 7.0)
        dA = torch.full((B, H, L), float("nan"), device=DEV)
        _btp.forward(c, xv, yv, ck, k, 32, flags=0)
        _btp.forward(c, xv, y32, ck, k, 32, flags=0)
        _btp.backward(c, xv, gv, ck, dxv, dA, k, 32)
        dx32 = torch.empty(shape, device=DEV, dtype=torch.float32)
        dA32 = torch.empty(B, H, L, device=DEV)
        _btp.backward(c, xv, gv, ck, dx32, dA32, k, 32, flags=_btp.FLAG_DX_F32)
        torch.cuda.synchronize()
        untouched("y", by, offsets[2])
        untouched("y fp32", by32, offsets[2] // 2)
        untouched("dx", bd, offsets[3])
        assert torch.equal(yv, y32.to(x.dtype)) and torch.equal(dxv, dx32.to(x.dtype)) and torch.equal(dA, dA32)
        ry = orc.forward(f64(coeff), f64(x), k=k)
        rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy), k=k)
        assert_close(f64(y32.cpu()), ry, F32_ATOL, F32_RTOL, "y fp32")
        assert_close(f64(yv.cpu()), ry, BF16_ATOL, BF16_RTOL, "y")
        assert_close(f64(dxv.cpu()), rdx, BF16_ATOL, BF16_RTOL, "dx")
        assert_close(f64(dA.cpu()), rdA, F32_ATOL, F32_RTOL, "dA")

        # fp32 dy holding the same values: the same arithmetic, dy moved the plain way
        (bd2, dx2), dA2 = _carve(shape, x.dtype, offsets[3], 7.0), torch.empty(B, H, L, device=DEV)
        _btp.backward(c, xv, gv32, ck, dx2, dA2, k, 32)
        torch.cuda.synchronize()
        untouched("dx (fp32 dy)", bd2, offsets[3])
        assert torch.equal(dx2, dxv) and torch.equal(dA2, dA)

        # log-space gates: y and dx to the 16-bit bound, dgate = a * dA
        (by3, y3), (bd3, dx3) = _carve(shape, x.dtype, offsets[2], 7.0), _carve(shape, x.dtype, offsets[3], 7.0)
        dgate = torch.empty(B, H, L, device=DEV)
        _btp.forward_log(gate, xv, y3, k)
        _btp.backward_log(gate, xv, gv, dx3, dgate, k)
        torch.cuda.synchronize()
        untouched("y (log gates)", by3, offsets[2])
        untouched("dx (log gates)", bd3, offsets[3])
        assert_close(f64(y3.cpu()), ry, BF16_ATOL, BF16_RTOL, "y (log gates)")
        assert_close(f64(dx3.cpu()), rdx, BF16_ATOL, BF16_RTOL, "dx (log gates)")
        assert_close(f64(dgate.cpu()), rdA * f64(coeff), 2 * F32_ATOL, 2 * F32_RTOL, "dgate")
    # the carries written beside y do not depend on how y moves
    y_ck, carries = run_forward(coeff, x, k=2, checkpoint=True)
    assert torch.equal(y_ck, run_forward(coeff, x, k=2))
    nb = L // 16
    rck = orc.forward(f64(coeff), f64(x), with_checkpoint=True)[1]
    assert_close(f64(carries)[:, :, : nb - 1], rck[:, :, : nb - 1], F32_ATOL, F32_RTOL, "checkpoint")


@pytest.mark.parametrize("L", [16, 32, 48, 64, 144, 160, 192, 288, 320, 576])
@pytest.mark.parametrize("B,H", [(1, 1), (1, 3), (2, 3), (1, 7), (5, 5), (8, 33)])
def test_spans_cut_from_the_block_sequence_of_the_tensor(B, H, L):
    """Rows that would leave a span partly empty (at most 64 steps; a few spans with little in the last one) have
    their spans cut from the blocks of all rows in order: short rows share a wavefront, longer ones start anywhere
    in one, and carries stop at the row starts. Every instance against the oracle, nothing written outside the
    tensors, and every row of the batch bit-identical to the same row run alone (where it starts its first span)."""
    from spear_amd import _btp

    coeff, x, dy = make_inputs(B, H, L, seed=700 + L + B * H, stress=1.5)
    c = coeff.to(DEV)
    gate = torch.log(c.float())
    shape = (B, H, 16, L)
    n = int(np.prod(shape))
    ck = torch.empty(0, device=DEV, dtype=torch.float32)
    xv, gv, gv32 = x.to(DEV), dy.to(DEV), dy.float().to(DEV)

    def untouched(name, buf, off=8):
        assert bool((buf[:off] == 7).all()) and bool((buf[off + n :] == 7).all()), f"{name}: bytes outside the tensor changed"

    for k in (2, 1):
        print(f"flat spans B={B} H={H} L={L} k={k}", flush=True)
        (by, yv), (bd, dxv) = _carve(shape, x.dtype, 8, 7.0), _carve(shape, x.dtype, 8, 7.0)
        (by32, y32), (bd32, dx32) = _carve(shape, torch.float32, 8, 7.0), _carve(shape, torch.float32, 8, 7.0)
        dA, dA32 = torch.full((B, H, L), float("nan"), device=DEV), torch.full((B, H, L), float("nan"), device=DEV)
        _btp.forward(c, xv, yv, ck, k, 32, flags=0)
        _btp.forward(c, xv, y32, ck, k, 32, flags=0)
        _btp.backward(c, xv, gv, ck, dxv, dA, k, 32)
        _btp.backward(c, xv, gv, ck, dx32, dA32, k, 32, flags=_btp.FLAG_DX_F32)
        torch.cuda.synchronize()
        for name, buf in (("y", by), ("y fp32", by32), ("dx", bd), ("dx fp32", bd32)):
            untouched(name, buf)
        assert torch.equal(yv, y32.to(x.dtype)) and torch.equal(dxv, dx32.to(x.dtype)) and torch.equal(dA, dA32)
        ry = orc.forward(f64(coeff), f64(x), k=k)
        rdx, rdA = orc.backward(f64(coeff), f64(x), f64(dy), k=k)
        assert_close(f64(y32.cpu()), ry, F32_ATOL, F32_RTOL, "y fp32")
        assert_close(f64(dx32.cpu()), rdx, F32_ATOL, F32_RTOL, "dx fp32")
        assert_close(f64(dA.cpu()), rdA, F32_ATOL, F32_RTOL, "dA")

        # fp32 dy with the same values; log-space gates
        dx2, dA2 = torch.empty_like(dxv), torch.empty_like(dA)
        _btp.backward(c, xv, gv32, ck, dx2, dA2, k, 32)
        assert torch.equal(dx2, dxv) and torch.equal(dA2, dA)
        y3, dx3, dgate = torch.empty_like(yv), torch.empty_like(dxv), torch.empty_like(dA)
        _btp.forward_log(gate, xv, y3, k)
        _btp.backward_log(gate, xv, gv, dx3, dgate, k)
        assert_close(f64(y3.cpu()), ry, BF16_ATOL, BF16_RTOL, "y (log gates)")
        assert_close(f64(dx3.cpu()), rdx, BF16_ATOL, BF16_RTOL, "dx (log gates)")
        assert_close(f64(dgate.cpu()), rdA * f64(coeff), 2 * F32_ATOL, 2 * F32_RTOL, "dgate")

        # rows alone
        for b, h in {(0, 0), (B - 1, H - 1), (B // 2, H // 2), (0, H - 1)}:
            c1, x1, g1 = (t[b : b + 1, h : h + 1].contiguous() for t in (c, xv, gv))
            y1, d1, a1 = torch.empty_like(x1), torch.empty_like(x1), torch.empty(1, 1, L, device=DEV)
            _btp.forward(c1, x1, y1, ck, k, 32, flags=0)
            _btp.backward(c1, x1, g1, ck, d1, a1, k, 32)
            assert torch.equal(y1, yv[b : b + 1, h : h + 1]) and torch.equal(d1, dxv[b : b + 1, h : h + 1])
            assert torch.equal(a1, dA[b : b + 1, h : h + 1]), f"row ({b}, {h}) differs from the same row run alone"
    # with the carry store the spans are cut per row: same y, carries against the oracle
    y_ck, carries = run_forward(coeff, x, k=2, checkpoint=True)
    assert torch.equal(y_ck, run_forward(coeff, x, k=2))
    nb = L // 16
    if nb > 1:
        rck = orc.forward(f64(coeff), f64(x), with_checkpoint=True)[1]
        assert_close(f64(carries)[:, :, : nb - 1], rck[:, :, : nb - 1], F32_ATOL, F32_RTOL, "checkpoint")


def test_kernels_match_the_reference_float64_path_vectors():
    """Forward and backward kernels against y, dx, dA computed by the reference's own float64 path and
    autograd (tests/golden/make_cpu_path_vectors.py)."""
    import pathlib

    v = np.load(pathlib.Path(__file__).with_name("golden") / "cpu_path_reference_vectors.npz")
    coeff, x, dy = (torch.from_numpy(v[n]).bfloat16() for n in ("a", "x", "dy"))
    assert_close(f64(run_forward(coeff, x)), v["ref.f64"], BF16_ATOL, BF16_RTOL, "y bf16")
    assert_close(f64(run_forward(coeff, x, out_dtype=torch.float32)), v["ref.f64"], F32_ATOL, F32_RTOL, "y fp32")
    dx, dA = run_backward(coeff, x, dy)
    assert_close(f64(dx), v["ref.f64.dx"], BF16_ATOL, BF16_RTOL, "dx")
    assert_close(f64(dA), v["ref.f64.dA"], F32_ATOL, F32_RTOL, "dA")


@pytest.mark.parametrize("slabs", [1, 3, 4, 1025])
def test_measurement_aids_move_the_bytes_they_are_timed_for(slabs):
    """spear_btp_copy and spear_btp_stream_probe are timed as ceilings, so they must really move every byte."""
    import ctypes

    from spear_amd import _btp

    lib = _btp.load_library()
    n = slabs * 4096
    g = torch.Generator(device="cpu").manual_seed(slabs)
    a = torch.randint(0, 256, (n,), dtype=torch.uint8, generator=g).to(DEV)
    b = torch.randint(0, 256, (n,), dtype=torch.uint8, generator=g).to(DEV)
    guard = 4096
    out = torch.full((n + guard,), 0xA5, dtype=torch.uint8, device=DEV)
    sp = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for second, want in ((None, a), (b, a ^ b)):
        out.fill_(0xA5)
        rc = lib.spear_btp_stream_probe(a.data_ptr(), None if second is None else second.data_ptr(), out.data_ptr(),
                                        ctypes.c_ulonglong(n), sp)
        assert rc == 0, lib.spear_btp_last_error()
        torch.cuda.synchronize()
        assert torch.equal(out[:n], want)
        assert bool((out[n:] == 0xA5).all())
    for shape in range(5):  # the alternative launch shapes of the probe move the same bytes
        for second, want in ((None, a), (b, a ^ b)):
            out.fill_(0xA5)
            rc = lib.spear_btp_stream_probe_shape(a.data_ptr(), None if second is None else second.data_ptr(),
                                                  out.data_ptr(), ctypes.c_ulonglong(n), shape, sp)
            assert rc == 0, lib.spear_btp_last_error()
            torch.cuda.synchronize()
            assert torch.equal(out[:n], want), shape
            assert bool((out[n:] == 0xA5).all()), shape
    # one-way shapes: 5 reads only and leaves dst alone, 6 writes every byte of dst and nothing beyond
    out.fill_(0xA5)
    assert lib.spear_btp_stream_probe_shape(a.data_ptr(), b.data_ptr(), out.data_ptr(), ctypes.c_ulonglong(n), 5, sp) == 0
    torch.cuda.synchronize()
    assert bool((out == 0xA5).all())
    assert lib.spear_btp_stream_probe_shape(a.data_ptr(), None, out.data_ptr(), ctypes.c_ulonglong(n), 6, sp) == 0
    torch.cuda.synchronize()
    words = out[:n].view(torch.int32).view(slabs, 4, 64, 4)
    assert bool((words[..., 1] == torch.arange(64, device=DEV, dtype=torch.int32).view(1, 1, 64)).all())
    assert bool((words[..., 0] == torch.arange(slabs, device=DEV, dtype=torch.int32).view(slabs, 1, 1)).all())
    assert bool((out[n:] == 0xA5).all())
    out.fill_(0xA5)  # shape 7: the 2R:1W combine, up to the lowest bit of every fourth word of a lane's last 16 bytes
    assert lib.spear_btp_stream_probe_shape(a.data_ptr(), b.data_ptr(), out.data_ptr(), ctypes.c_ulonglong(n), 7, sp) == 0
    torch.cuda.synchronize()
    diff = (out[:n] ^ (a ^ b)).view(torch.int32)
    assert bool(((diff & ~1) == 0).all()) and bool((out[n:] == 0xA5).all())
    assert lib.spear_btp_stream_probe_shape(a.data_ptr(), None, out.data_ptr(), ctypes.c_ulonglong(n), 8, sp) == -1
    # the probe with several inputs and outputs: every output is the combination of all inputs, nothing beyond
    ins = [a, b, a.flip(0).contiguous(), b.flip(0).contiguous()]
    outs = [torch.full((n + guard,), 0xA5, dtype=torch.uint8, device=DEV) for _ in range(3)]
    for n_src, n_dst in ((3, 1), (4, 3), (1, 2)):
        want = ins[0]
        for t in ins[1:n_src]:
            want = want ^ t
        for compute in (0, 1):
            for o in outs:
                o.fill_(0xA5)
            src = (ctypes.c_void_p * n_src)(*[t.data_ptr() for t in ins[:n_src]])
            dst = (ctypes.c_void_p * n_dst)(*[t.data_ptr() for t in outs[:n_dst]])
            assert lib.spear_btp_stream_probe_mix(src, n_src, dst, n_dst, ctypes.c_ulonglong(n), compute, sp) == 0
            torch.cuda.synchronize()
            for o in outs[:n_dst]:
                diff = (o[:n] ^ want).view(torch.int32)
                assert bool(((diff & ~compute) == 0).all()) and bool((o[n:] == 0xA5).all()), (n_src, n_dst, compute)
            for o in outs[n_dst:]:
                assert bool((o == 0xA5).all())
    src2 = (ctypes.c_void_p * 2)(a.data_ptr(), b.data_ptr())
    dst1 = (ctypes.c_void_p * 1)(outs[0].data_ptr())
    assert lib.spear_btp_stream_probe_mix(src2, 2, dst1, 1, ctypes.c_ulonglong(n), 0, sp) == -1
    out.fill_(0xA5)
    assert lib.spear_btp_copy(a.data_ptr(), out.data_ptr(), ctypes.c_ulonglong(n), sp) == 0
    torch.cuda.synchronize()
    assert torch.equal(out[:n], a) and bool((out[n:] == 0xA5).all())


def test_concurrent_callers_on_their_own_streams():
    """The library keeps no state between calls (the error string is per thread): two host threads
    launching on two streams at once get the results they get alone."""
    import threading

    from spear_amd import _btp

    cases = []
    for seed in (501, 502):
        coeff, x, dy = make_inputs(8, 8, 1024, seed=seed)
        cases.append([t.to(DEV) for t in (coeff, x, dy)])
    alone = [(run_forward(c.cpu(), x.cpu()), run_backward(c.cpu(), x.cpu(), g.cpu())) for c, x, g in cases]
    results, errors = [None, None], []

    def worker(i):
        try:
            c, x, g = cases[i]
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(25):
                    y = torch.empty_like(x)
                    dx = torch.empty_like(x)
                    dA = torch.empty(c.shape, device=DEV, dtype=torch.float32)
                    ck = torch.empty(8, 8, 64, 16, device=DEV, dtype=torch.float32)
                    _btp.forward(c, x, y, ck, 2, 32, flags=0)
                    _btp.backward(c, x, g, ck, dx, dA, 2, 32)
                stream.synchronize()
            results[i] = (y.cpu(), dx.cpu(), dA.cpu())
        except Exception as e:  # surfaced below: an exception in a thread would otherwise pass silently
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for (y, dx, dA), (y0, (dx0, dA0)) in zip(results, alone):
        assert torch.equal(y, y0) and torch.equal(dx, dx0) and torch.equal(dA, dA0)
