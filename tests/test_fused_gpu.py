"""The fused layer-layout forward (spear_phalanx_mix_forward / phalanx_mix / Phalanx(method="fused"))
against the float64 composition of the pinned BTP oracle with sigmoid gates, and against the
unfused HIP path of the layer."""

import numpy as np
import pytest
import torch

from helpers import BF16_ATOL, BF16_RTOL, assert_close, f64
from oracle import btp_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make_mix_inputs(B, L, H, Hkv, seed, dtype=torch.bfloat16, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    a = (torch.randn(B, L, H, generator=g) * scale).to(dtype)
    b = (torch.randn(B, L, Hkv * 16, generator=g) * scale).to(dtype)
    c = torch.randn(B, L, Hkv * 16, generator=g).to(dtype)
    v = torch.randn(B, L, H * 16, generator=g).to(dtype)
    return a, b, c, v


def run_mix(a, b, c, v, H, Hkv):
    from spear_amd import _btp

    out = torch.full(v.shape, float("nan"), device=DEV, dtype=v.dtype)
    _btp.mix_forward(a.to(DEV), b.to(DEV), c.to(DEV), v.to(DEV), out, H, Hkv)
    torch.cuda.synchronize()
    return out.cpu()


# head counts and groupings as the reference's KVRepeat accepts them (spear/nn/phalanx/swr.py:37-38: any
# heads % kv_heads == 0): head counts that do not fill a wavefront's 8 heads or are odd (gate logits then do not pair
# up into aligned 32-bit words), groups of 1, 2, 4, 8 heads per kv head (summed inside a wavefront in backward) and
# every other group size (3, 5, 6, 7: whole groups per wavefront; 12, 16, 20, 24, 32: worked through 8 heads at a time)
ODD_GROUPINGS = [(2, 48, 6, 3), (1, 80, 12, 12), (2, 64, 3, 1), (1, 32, 1, 1), (2, 96, 5, 5), (1, 144, 10, 2),
                 (2, 64, 16, 1), (1, 80, 32, 2), (2, 48, 6, 2), (1, 112, 12, 2), (2, 64, 7, 1), (1, 272, 12, 1),
                 (1, 64, 24, 1), (2, 80, 40, 2), (1, 48, 9, 3), (3, 64, 36, 6), (1, 2064, 16, 1)]


@pytest.mark.parametrize("B,L,H,Hkv", [
    (1, 16, 4, 4), (2, 32, 4, 4), (2, 48, 8, 8), (1, 80, 4, 2), (3, 128, 8, 2), (2, 144, 16, 4),
    (1, 512, 32, 32), (2, 272, 12, 3), (1, 1040, 4, 1), (1, 4096, 8, 8), (2, 2064, 16, 2),
    (5, 64, 32, 8), (3, 272, 128, 16),
    # grids beyond one window of the dealing of workgroups to XCDs (1024 workgroups), with a tail
    # that keeps the launch order: 1096 and 1500 workgroups
    (137, 128, 32, 32), (100, 272, 24, 8),
] + ODD_GROUPINGS)
def test_fused_forward_matches_oracle(B, L, H, Hkv):
    a, b, c, v = make_mix_inputs(B, L, H, Hkv, seed=1000 + L + H)
    print(f"fused B={B} L={L} H={H} Hkv={Hkv}", flush=True)
    out = run_mix(a, b, c, v, H, Hkv)
    ref = orc.phalanx_mix_forward(f64(a), f64(b), f64(c), f64(v), H, Hkv)
    assert_close(f64(out), ref, BF16_ATOL, BF16_RTOL, "out")


def test_fused_forward_fp16_and_steep_gates():
    a, b, c, v = make_mix_inputs(2, 96, 8, 4, seed=5, dtype=torch.float16, scale=4.0)
    a[0, :10, :] = -30.0  # decay ~ 1e-13: counts as zero
    a[1, 20:40, 3] = 30.0  # decay -> 1
    out = run_mix(a, b, c, v, 8, 4)
    ref = orc.phalanx_mix_forward(f64(a), f64(b), f64(c), f64(v), 8, 4)
    assert_close(f64(out), ref, 4e-3, 4e-3, "out fp16")


def run_mix_backward(a, b, c, v, dout, H, Hkv=None):
    from spear_amd import _btp

    dev = [t.to(DEV) for t in (a, b, c, v, dout)]
    outs = [torch.full(t.shape, float("nan"), device=DEV, dtype=t.dtype) for t in (a, b, c, v)]
    _btp.mix_backward(*dev, *outs, H, H if Hkv is None else Hkv)
    torch.cuda.synchronize()
    return [t.cpu() for t in outs]


@pytest.mark.parametrize("B,L,H", [(1, 16, 4), (2, 32, 4), (2, 48, 8), (1, 80, 12), (3, 128, 8), (2, 144, 16), (1, 512, 32), (1, 1040, 4), (1, 4096, 8), (2, 2064, 16),
                                   (5, 64, 32), (2, 112, 24), (3, 272, 64),
                                   # grids beyond one window of the dealing of workgroups to XCDs (1024
                                   # workgroups), with a tail that keeps the launch order: 1096 and 1500 workgroups
                                   (137, 128, 32), (100, 272, 24)])
def test_fused_backward_matches_oracle(B, L, H):
    a, b, c, v = make_mix_inputs(B, L, H, H, seed=2000 + L + H)
    dout = torch.randn(B, L, H * 16, generator=torch.Generator().manual_seed(L)).bfloat16()
    print(f"fused bwd B={B} L={L} H={H}", flush=True)
    da, db, dc, dv = run_mix_backward(a, b, c, v, dout, H)
    rda, rdb, rdc, rdv = orc.phalanx_mix_backward(f64(a), f64(b), f64(c), f64(v), f64(dout), H, H)
    assert_close(f64(dv), rdv, BF16_ATOL, BF16_RTOL, "dv")
    assert_close(f64(dc), rdc, BF16_ATOL, BF16_RTOL, "dc")
    assert_close(f64(db), rdb, BF16_ATOL, BF16_RTOL, "db")
    assert_close(f64(da), rda, BF16_ATOL, BF16_RTOL, "da")


@pytest.mark.parametrize("B,L,H,Hkv", [(2, 48, 8, 4), (1, 80, 12, 3), (2, 144, 16, 2), (1, 272, 32, 8), (2, 64, 4, 2),
                                       (1, 2064, 8, 1)] + ODD_GROUPINGS)
def test_fused_backward_with_shared_kv_heads(B, L, H, Hkv):
    """Every head grouping at the bf16 bound: the sums over a group are taken in fp32 and rounded once."""
    a, b, c, v = make_mix_inputs(B, L, H, Hkv, seed=3000 + L + H)
    dout = torch.randn(B, L, H * 16, generator=torch.Generator().manual_seed(L + 1)).bfloat16()
    print(f"fused bwd kv B={B} L={L} H={H} Hkv={Hkv}", flush=True)
    da, db, dc, dv = run_mix_backward(a, b, c, v, dout, H, Hkv)
    rda, rdb, rdc, rdv = orc.phalanx_mix_backward(f64(a), f64(b), f64(c), f64(v), f64(dout), H, Hkv)
    assert_close(f64(dv), rdv, BF16_ATOL, BF16_RTOL, "dv")
    assert_close(f64(dc), rdc, BF16_ATOL, BF16_RTOL, "dc")
    assert_close(f64(db), rdb, BF16_ATOL, BF16_RTOL, "db")
    assert_close(f64(da), rda, BF16_ATOL, BF16_RTOL, "da")
    # a second run gives the same bits: every sum is taken in a fixed order
    again = run_mix_backward(a, b, c, v, dout, H, Hkv)
    for x, y in zip((da, db, dc, dv), again):
        assert torch.equal(x, y)


@pytest.mark.parametrize("B,L,H,Hkv", [(1, 16, 4, 4), (3, 128, 8, 8), (2, 144, 16, 2), (1, 80, 12, 3), (1, 272, 32, 4),
                                       (2, 2064, 8, 1), (40, 64, 32, 32), (1, 8192, 8, 8), (3, 112, 128, 16),
                                       (70, 272, 32, 32), (2, 80, 6, 2), (1, 144, 16, 1), (3, 48, 40, 2), (2, 64, 7, 7),
                                       (1, 96, 12, 1), (2, 64, 10, 2)])
def test_fused_backward_column_sums_match_oracle(B, L, H, Hkv):
    """The partial sums the backward kernel leaves (one row per batch row and tile of 64 time steps) add up to the
    oracle's gradients summed over batch and time (the bias gradients of proj_a, proj_b, proj_c); the gradients
    themselves are unchanged by asking."""
    from spear_amd import _btp

    a, b, c, v = make_mix_inputs(B, L, H, Hkv, seed=5000 + L + H)
    dout = torch.randn(B, L, H * 16, generator=torch.Generator().manual_seed(L + 2)).bfloat16()
    print(f"fused bwd sums B={B} L={L} H={H} Hkv={Hkv}", flush=True)
    plain = run_mix_backward(a, b, c, v, dout, H, Hkv)
    dev = [t.to(DEV) for t in (a, b, c, v, dout)]
    outs = [torch.full(t.shape, float("nan"), device=DEV, dtype=t.dtype) for t in (a, b, c, v)]
    rows = _btp.mix_backward_sum_rows(B, L, H)
    assert rows == B * -(-(L // 16) // 4)
    sums = tuple(torch.full((rows, w), float("nan"), device=DEV) for w in (H, Hkv * 16, Hkv * 16))
    _btp.mix_backward(*dev, *outs, H, Hkv, sums=sums)
    torch.cuda.synchronize()
    for got, want in zip(outs, plain):
        assert torch.equal(got.cpu(), want)
    rda, rdb, rdc, _ = orc.phalanx_mix_backward(f64(a), f64(b), f64(c), f64(v), f64(dout), H, Hkv)
    for name, s, ref in (("da", sums[0], rda), ("db", sums[1], rdb), ("dc", sums[2], rdc)):
        got = f64(s.cpu()).sum(0)
        want, mass = ref.sum((0, 1)), np.abs(ref).sum((0, 1))
        # fp32 arithmetic on bf16 inputs; the sums are taken before any rounding to bf16
        assert np.all(np.abs(got - want) <= 2e-4 * mass + 1e-5), (name, np.abs(got - want).max(), mass.max())
    with pytest.raises(RuntimeError, match="shape"):
        _btp.mix_backward(*dev, *outs, H, Hkv,
                          sums=tuple(torch.empty(rows + 1, w, device=DEV) for w in (H, Hkv * 16, Hkv * 16)))


@pytest.mark.parametrize("B,L,H,Hkv", [(1, 16, 4, 4), (3, 128, 8, 8), (2, 144, 16, 2), (1, 80, 12, 3), (2, 2064, 8, 1), (40, 64, 32, 32),
                                       (2, 48, 6, 2), (1, 80, 16, 1), (2, 64, 5, 5)])
def test_fused_backward_into_column_blocks_of_one_buffer(B, L, H, Hkv):
    """The four gradients written side by side into one [B, L, ld] buffer are bit-identical to the dense
    ones, and the columns between and after the blocks are left alone."""
    from spear_amd import _btp
    from spear_amd.nn.phalanx.projections import packed_columns

    a, b, c, v = make_mix_inputs(B, L, H, Hkv, seed=6000 + L + H)
    dout = torch.randn(B, L, H * 16, generator=torch.Generator().manual_seed(L + 3)).bfloat16()
    print(f"fused bwd packed B={B} L={L} H={H} Hkv={Hkv}", flush=True)
    plain = run_mix_backward(a, b, c, v, dout, H, Hkv)
    cols, ld = packed_columns(H, Hkv)
    assert ld % 64 == 0 and ld >= cols["a"][0] + cols["a"][1]
    ld += 64                                              # more slack than needed, so there is padding to check
    dev = [t.to(DEV) for t in (a, b, c, v, dout)]
    marker = 12345.0
    packed = torch.full((B, L, ld), marker, device=DEV, dtype=torch.bfloat16)
    views = [packed[..., cols[k][0]:cols[k][0] + cols[k][1]] for k in "abcv"]
    _btp.mix_backward(*dev, *views, H, Hkv)
    torch.cuda.synchronize()
    for got, want in zip(views, plain):
        assert torch.equal(got.cpu(), want)
    used = cols["a"][0] + cols["a"][1]
    assert bool((packed[..., used:] == marker).all())
    # a block that is not a column block of a dense buffer is refused
    with pytest.raises(RuntimeError, match="column block"):
        every_other = torch.empty(B, L, 2 * H * 16, device=DEV, dtype=torch.bfloat16)[..., ::2]
        _btp.mix_backward(*dev, views[0], views[1], views[2], every_other, H, Hkv)


def test_fused_backward_fp16_and_steep_gates():
    a, b, c, v = make_mix_inputs(2, 96, 8, 4, seed=6, dtype=torch.float16, scale=3.0)
    a[0, :10, :] = -30.0  # decay ~ 1e-13: counts as zero
    a[1, 20:40, 3] = 30.0  # decay -> 1
    dout = torch.randn(2, 96, 128, generator=torch.Generator().manual_seed(7)).half()
    da, db, dc, dv = run_mix_backward(a, b, c, v, dout, 8, 4)
    rda, rdb, rdc, rdv = orc.phalanx_mix_backward(f64(a), f64(b), f64(c), f64(v), f64(dout), 8, 4)
    # fp16 storage: 11 significant bits; sums over two heads and up to 32 steps of undamped states
    for name, got, want in (("dv", dv, rdv), ("dc", dc, rdc), ("db", db, rdb), ("da", da, rda)):
        assert_close(f64(got), want, 2e-2, 4e-3, name + " fp16")


@pytest.mark.parametrize("H,Hkv", [(8, 4), (16, 1), (32, 2), (6, 3), (12, 12), (6, 2)])
def test_fused_op_autograd_matches_unfused_composition(H, Hkv):
    """Gradients of phalanx_mix against autograd through the same composition built from torch ops
    and the float64 reference recurrence, at the bf16 bound for every head grouping."""
    from spear_amd import phalanx_mix
    from spear_amd.ops.btp.reference import block_two_pass_ref

    B, L = 2, 64
    a, b, c, v = make_mix_inputs(B, L, H, Hkv, seed=21)
    dout = torch.randn(B, L, H * 16, generator=torch.Generator().manual_seed(22)).bfloat16()

    leaves = [t.clone().to(DEV).requires_grad_(True) for t in (a, b, c, v)]
    out = phalanx_mix(*leaves, heads=H, kv_heads=Hkv)
    out.backward(dout.to(DEV))

    ref_leaves = [t.clone().double().requires_grad_(True) for t in (a, b, c, v)]
    ra, rb, rc, rv = ref_leaves
    g = H // Hkv
    heads = lambda t, h: t.view(B, L, h, 16).permute(0, 2, 3, 1)
    A = torch.sigmoid(ra).transpose(1, 2)
    G = torch.sigmoid(heads(rb, Hkv)).repeat_interleave(g, 1)
    C = heads(rc, Hkv).repeat_interleave(g, 1)
    V = heads(rv, H)
    hh = block_two_pass_ref(A.contiguous(), (G * V).contiguous())
    ref_out = (hh * C + V).permute(0, 3, 1, 2).reshape(B, L, H * 16)
    ref_out.backward(dout.double())

    assert_close(f64(out), ref_out.detach().numpy(), BF16_ATOL, BF16_RTOL, "out")
    for name, got, want in zip("abcv", leaves, ref_leaves):
        assert_close(f64(got.grad), want.grad.numpy(), BF16_ATOL, BF16_RTOL, f"d{name}")


def test_phalanx_fused_method_matches_default_and_pytorch():
    from spear_amd import Phalanx
    from spear_amd.testing.numerics import compute_error_metrics

    torch.manual_seed(0)
    ref = Phalanx(dim=512, length=128, method="pytorch", dtype=torch.bfloat16)
    fused = Phalanx(dim=512, length=128, method="fused", dtype=torch.bfloat16).to(DEV)
    dflt = Phalanx(dim=512, length=128, method="default", dtype=torch.bfloat16).to(DEV)
    fused.load_state_dict(ref.state_dict())
    dflt.load_state_dict(ref.state_dict())
    x = torch.randn(8, 128, 512, generator=torch.Generator().manual_seed(1)).bfloat16()
    y_ref, y_f, y_d = ref(x), fused(x.to(DEV)).cpu(), dflt(x.to(DEV)).cpu()
    for name, y in (("fused", y_f), ("default", y_d)):
        m = compute_error_metrics(y, y_ref)
        assert m["max_abs"] <= 1e-1 and m["rmse"] <= 5e-2, (name, m)  # layer forward limits of the reference tests
    assert_close(f64(y_f), f64(y_ref), 2e-2, 2e-2, "fused layer y")

    # and it trains: gradients reach every parameter
    fused.zero_grad()
    fused(x.to(DEV)).float().square().mean().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad.float()).all() for p in fused.parameters())


def test_fused_method_needs_k_2_and_takes_every_head_count():
    from spear_amd import Phalanx

    with pytest.raises(ValueError, match="k == 2"):
        Phalanx(dim=128, method="fused", dtype=torch.bfloat16, k=1)
    for dim, kv_heads in ((96, None), (96, 2), (48, 1), (256, 1)):  # 6 heads, groups of 3, 3 heads shared, groups of 16
        torch.manual_seed(5)
        ref = Phalanx(dim=dim, length=64, method="pytorch", dtype=torch.bfloat16, kv_heads=kv_heads)
        fused = Phalanx(dim=dim, length=64, method="fused", dtype=torch.bfloat16, kv_heads=kv_heads).to(DEV)
        fused.load_state_dict(ref.state_dict())
        x = torch.randn(2, 64, dim, generator=torch.Generator().manual_seed(6)).bfloat16()
        assert_close(f64(fused(x.to(DEV))), f64(ref(x)), 2e-2, 2e-2, f"fused layer y, dim {dim} kv_heads {kv_heads}")
        fused.zero_grad()
        fused(x.to(DEV)).float().square().mean().backward()
        assert all(p.grad is not None and torch.isfinite(p.grad.float()).all() for p in fused.parameters())


def test_default_method_rerouted_by_environment_gives_the_fused_results(monkeypatch):
    from spear_amd import Phalanx

    torch.manual_seed(3)
    fused = Phalanx(dim=128, length=64, method="fused", dtype=torch.bfloat16).to(DEV)
    monkeypatch.setenv("SPEAR_PHALANX_DEFAULT", "fused")
    rerouted = Phalanx(dim=128, length=64, dtype=torch.bfloat16).to(DEV)
    rerouted.load_state_dict(fused.state_dict())
    x = torch.randn(2, 64, 128, generator=torch.Generator().manual_seed(4)).bfloat16().to(DEV)
    assert torch.equal(rerouted(x), fused(x))


@pytest.mark.parametrize("H,Hkv", [(16, 4), (12, 2), (16, 1)])
def test_qkv_form_backward_against_the_oracle(H, Hkv):
    """The q/k/v/gate form of the backward kernel, with groups summed inside a wavefront and through LDS."""
    from spear_amd import _btp

    B, L = 3, 176
    g = torch.Generator().manual_seed(8102)
    gate = -torch.nn.functional.softplus(torch.randn(B, L, H, generator=g))
    q, k, vv, dd = ((0.5 * torch.randn(B, L, w, generator=g)).bfloat16() for w in (Hkv * 16, Hkv * 16, H * 16, H * 16))
    outs = [torch.full(t.shape, float("nan"), device=DEV, dtype=t.dtype) for t in (gate, k, q, vv)]
    _btp.mix_backward(gate.to(DEV), k.to(DEV), q.to(DEV), vv.to(DEV), dd.to(DEV), *outs, H, Hkv, qkv_gate=True)
    torch.cuda.synchronize()
    rgate, rk, rq, rv = orc.qkv_gate_backward(f64(q), f64(k), f64(vv), f64(gate), f64(dd), H, Hkv)
    assert_close(f64(outs[0]), rgate, 1e-4, 1e-4, "dgate")
    assert_close(f64(outs[1]), rk, BF16_ATOL, BF16_RTOL, "dk")
    assert_close(f64(outs[2]), rq, BF16_ATOL, BF16_RTOL, "dq")
    assert_close(f64(outs[3]), rv, BF16_ATOL, BF16_RTOL, "dv")
