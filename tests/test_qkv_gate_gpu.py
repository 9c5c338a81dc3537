"""The fused kernels in q/k/v/gate terms (SPEAR_MIX_QKV_GATE, ``spear_amd.btp_qkv``):
out = q * btp(exp(gate), k * v) + v on time-major [B, L, H, 16] tensors with an fp32 log-decay gate,
and dq, dk, dv, dgate -- against the float64 composition of the pinned BTP oracle on the same
bf16-rounded inputs. Tolerance: 2e-2 absolute + relative for 16-bit results, and for dgate (fp32 storage,
fp32 arithmetic on bf16 operands) 1e-4 relative to the gradient's scale."""

import numpy as np
import pytest
import torch

from helpers import BF16_ATOL, BF16_RTOL, F32_ATOL, F32_RTOL, assert_close, f64
from oracle import btp_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make_qkv(B, L, H, Hkv, seed, dtype=torch.bfloat16, std=0.25, gates="softplus"):
    g = torch.Generator().manual_seed(seed)
    q = (std * torch.randn(B, L, Hkv, 16, generator=g)).to(dtype)
    k = (std * torch.randn(B, L, Hkv, 16, generator=g)).to(dtype)
    v = (std * torch.randn(B, L, H, 16, generator=g)).to(dtype)
    if gates == "softplus":
        gate = -torch.nn.functional.softplus(torch.randn(B, L, H, generator=g))
    else:  # per head: near-total forgetting or near-identity (the log-space stress of configuration 5)
        forget = torch.rand(H, generator=g) < 0.5
        u = torch.rand(B, L, H, generator=g)
        gate = torch.where(forget, -20.0 + 15.0 * u, -1e-4 * u)
    dout = torch.randn(B, L, H, 16, generator=g).to(dtype)
    return q, k, v, gate.float(), dout


def flat(t):
    return t.reshape(t.shape[0], t.shape[1], -1)


def run(q, k, v, gate, dout):
    from spear_amd import btp_qkv

    leaves = [t.to(DEV).requires_grad_(True) for t in (q, k, v, gate)]
    out = btp_qkv(*leaves)
    out.backward(dout.to(DEV))
    torch.cuda.synchronize()
    return out.detach().cpu(), [t.grad.cpu() for t in leaves]


def check(q, k, v, gate, dout, atol=BF16_ATOL, rtol=BF16_RTOL):
    H, Hkv = v.shape[2], q.shape[2]
    out, (dq, dk, dv, dgate) = run(q, k, v, gate, dout)
    assert out.shape == v.shape and out.dtype == v.dtype and dgate.dtype == torch.float32
    args = [f64(flat(t)) for t in (q, k, v)] + [f64(gate)]
    assert_close(f64(flat(out)), orc.qkv_gate_forward(*args, H, Hkv), atol, rtol, "out")
    rgate, rk, rq, rv = orc.qkv_gate_backward(*args, f64(flat(dout)), H, Hkv)
    assert_close(f64(flat(dv)), rv, atol, rtol, "dv")
    assert_close(f64(flat(dq)), rq, atol, rtol, "dq")  # sums over a head group: fp32, rounded once
    assert_close(f64(flat(dk)), rk, atol, rtol, "dk")
    scale = max(1.0, float(np.abs(rgate).max()))
    assert float(np.abs(f64(dgate) - rgate).max()) <= 1e-4 * scale, ("dgate", float(np.abs(f64(dgate) - rgate).max()), scale)


@pytest.mark.parametrize("B,L,H,Hkv", [(1, 16, 4, 4), (2, 48, 8, 8), (1, 80, 12, 3), (3, 128, 8, 2), (2, 144, 16, 16),
                                       (1, 512, 32, 32), (1, 1040, 4, 1), (2, 2064, 16, 2), (1, 4096, 8, 8),
                                       (2, 64, 6, 2), (1, 80, 16, 1), (2, 48, 5, 5), (1, 112, 24, 2)])
def test_qkv_gate_forward_and_backward_match_oracle(B, L, H, Hkv):
    print(f"qkv B={B} L={L} H={H} Hkv={Hkv}", flush=True)
    check(*make_qkv(B, L, H, Hkv, seed=7000 + L + H))


def test_gates_next_to_zero_and_next_to_minus_infinity():
    """fp32 log gates keep what a 16-bit linear decay cannot: exp(-1e-4 u) != 1, and exp(-20) is tiny but
    not treated as exactly 1 or 0 before its time."""
    check(*make_qkv(2, 272, 16, 16, seed=71, std=1.0, gates="mixed"))
    q, k, v, gate, dout = make_qkv(1, 64, 4, 4, seed=72)
    gate[0, 5:9] = -float("inf")     # decay exactly 0: the state is cut
    gate[0, 20:24] = 0.0             # decay exactly 1
    gate[0, 40] = -25.0              # below the kernels' 1e-9 floor: counts as 0
    out, (dq, dk, dv, dgate) = run(q, k, v, gate, dout)
    assert all(bool(torch.isfinite(t.float()).all()) for t in (out, dq, dk, dv, dgate))
    g2 = gate.clone()
    g2[0, 40] = -float("inf")
    args = [f64(flat(t)) for t in (q, k, v)] + [f64(g2)]
    assert_close(f64(flat(out)), orc.qkv_gate_forward(*args, 4, 4), BF16_ATOL, BF16_RTOL, "out with cut states")
    assert float(dgate[0, 5:9].abs().max()) == 0.0 and float(dgate[0, 40].abs().max()) == 0.0


def test_fp16_operands():
    q, k, v, gate, dout = make_qkv(2, 96, 8, 4, seed=73, dtype=torch.float16)
    check(q, k, v, gate, dout, atol=4e-3, rtol=4e-3)


def test_same_numbers_as_the_log_gate_operator_with_glue():
    """The fused form against the stand-alone log-gate kernels wrapped in PyTorch element-wise ops
    (the route a caller would take without it)."""
    from spear_amd import btp_log, btp_qkv

    q, k, v, gate, dout = make_qkv(4, 256, 16, 16, seed=74)
    qd, kd, vd, gd = (t.to(DEV) for t in (q, k, v, gate))
    out = btp_qkv(qd, kd, vd, gd)
    heads = lambda t: t.permute(0, 2, 3, 1).contiguous()                    # [B, L, H, 16] -> [B, H, 16, L]
    x = (heads(kd).float() * heads(vd).float()).to(torch.bfloat16)
    h = btp_log(gd.transpose(1, 2).contiguous(), x, output_dtype=torch.float32)
    want = (h * heads(qd).float() + heads(vd).float()).permute(0, 3, 1, 2)  # the glue rounds k*v to bf16 first
    err = (out.float() - want).abs() - (BF16_ATOL + BF16_RTOL * want.abs())
    assert float(err.max()) <= 0


# The benchmark configurations in the terms they are worded in (q, k, v bf16, fp32 log-decay gate; check out,
# dq, dk, dv, dgate), at full size: B1024 L128 H32 with gate = -softplus(N(0,1)) and q/k/v ~ N(0, 1/16); the long
# rows B16 L8192 H64; and B64 L2048 H128 with q/k/v ~ N(0,1) and per head either U[-20,-5] or U[-1e-4,0] gates.
BENCH_SHAPES = {
    "c3_B1024_L128_H32": dict(B=1024, L=128, H=32, seed=1234, std=0.25, gates="softplus"),
    "c4_B16_L8192_H64": dict(B=16, L=8192, H=64, seed=1235, std=0.25, gates="softplus"),
    "c5_B64_L2048_H128": dict(B=64, L=2048, H=128, seed=1236, std=1.0, gates="mixed"),
}


@pytest.mark.parametrize("name", list(BENCH_SHAPES))
def test_benchmark_shapes_forward_and_backward(name):
    """Full-size forward and backward; the oracle on sampled batch rows (rows are independent), and the
    properties that need no oracle: q = 0 returns v, a slice of the batch run alone gives the same bits."""
    from spear_amd import btp_qkv

    cfg = BENCH_SHAPES[name]
    B, L, H = cfg["B"], cfg["L"], cfg["H"]
    print(f"{name}: generating inputs", flush=True)
    q, k, v, gate, dout = make_qkv(B, L, H, H, seed=cfg["seed"], std=cfg["std"], gates=cfg["gates"])
    print(f"{name}: forward/backward", flush=True)
    leaves = [t.to(DEV).requires_grad_(True) for t in (q, k, v, gate)]
    out = btp_qkv(*leaves)
    out.backward(dout.to(DEV))
    torch.cuda.synchronize()
    qd, kd, vd, gd = (t.detach() for t in leaves)
    grads = [t.grad for t in leaves]
    assert all(bool(torch.isfinite(t.float()).all()) for t in (out, *grads))
    assert torch.equal(btp_qkv(torch.zeros_like(qd), kd, vd, gd), vd)     # q = 0 leaves v
    lo = B - 3
    part = [t[lo:].contiguous().requires_grad_(True) for t in (qd, kd, vd, gd)]
    out_part = btp_qkv(*part)
    out_part.backward(dout[lo:].to(DEV))
    assert torch.equal(out_part.detach(), out.detach()[lo:])
    for name_g, gp, gall in zip(("dq", "dk", "dv", "dgate"), part, grads):
        assert torch.equal(gp.grad, gall[lo:]), name_g

    print(f"{name}: oracle on sampled batch rows", flush=True)
    rng = np.random.default_rng(cfg["seed"])
    sample = sorted(set([0, B - 1] + [int(i) for i in rng.integers(0, B, size=2)]))
    args = [f64(flat(t[sample])) for t in (q, k, v)] + [f64(gate[sample])]
    assert_close(f64(flat(out.detach()[sample].cpu())), orc.qkv_gate_forward(*args, H, H), BF16_ATOL, BF16_RTOL, "out")
    rgate, rk, rq, rv = orc.qkv_gate_backward(*args, f64(flat(dout[sample])), H, H)
    dq, dk, dv, dgate = (t[sample].cpu() for t in grads)
    assert_close(f64(flat(dv)), rv, BF16_ATOL, BF16_RTOL, "dv")
    assert_close(f64(flat(dq)), rq, BF16_ATOL, BF16_RTOL, "dq")
    assert_close(f64(flat(dk)), rk, BF16_ATOL, BF16_RTOL, "dk")
    assert_close(f64(dgate), rgate, F32_ATOL, F32_RTOL, "dgate")


def test_log_gate_operator_at_the_log_space_stress_shape():
    """btp_log (fp32 log-space gates in the op's own [B, H, 16, L] layout) at B64 H128 L2048 with the per-head
    forgetting / near-identity mixture: y, dx, dgate on sampled rows against the oracle at a = exp(gate)."""
    from spear_amd import btp_log

    B, H, L = 64, 128, 2048
    g = torch.Generator().manual_seed(1236)
    print("btp_log c5: generating inputs", flush=True)
    forget = torch.rand(B, H, 1, generator=g) < 0.5
    u = torch.rand(B, H, L, generator=g)
    gate = torch.where(forget, -20.0 + 15.0 * u, -1e-4 * u).float()
    x = torch.randn(B, H, 16, L, generator=g).bfloat16()
    dy = torch.randn(B, H, 16, L, generator=g).bfloat16()
    gd, xd = gate.to(DEV).requires_grad_(True), x.to(DEV).requires_grad_(True)
    print("btp_log c5: forward/backward", flush=True)
    y = btp_log(gd, xd, output_dtype=torch.float32)
    y.backward(dy.to(DEV).float())
    torch.cuda.synchronize()
    assert all(bool(torch.isfinite(t.float()).all()) for t in (y, gd.grad, xd.grad))
    rng = np.random.default_rng(1236)
    rows = list(zip(rng.integers(0, B, size=6), rng.integers(0, H, size=6)))
    rows += [(int(b), int(h)) for b, h in zip(*np.nonzero(~forget[:, :, 0].numpy()))][:2]  # two near-identity heads for sure
    print("btp_log c5: oracle on sampled rows", flush=True)
    for b, h in rows:
        sl = (slice(b, b + 1), slice(h, h + 1))
        a = np.exp(f64(gate[sl]))
        ry = orc.forward(a, f64(x[sl]))
        rdx, rdA = orc.backward(a, f64(x[sl]), f64(dy[sl]))
        assert_close(f64(y.detach()[sl]), ry, F32_ATOL, F32_RTOL, f"y[{b},{h}]")
        assert_close(f64(xd.grad[sl]), rdx, BF16_ATOL, BF16_RTOL, f"dx[{b},{h}]")
        assert_close(f64(gd.grad[sl]), rdA * a, F32_ATOL, F32_RTOL, f"dgate[{b},{h}]")


def test_rejects_what_it_cannot_do():
    from spear_amd import _btp, btp_qkv

    q, k, v, gate, _ = make_qkv(1, 32, 16, 3, seed=76)
    with pytest.raises(RuntimeError, match="divisible by kv_heads"):
        btp_qkv(*(t.to(DEV) for t in (q, k, v, gate)))
    q, k, v, gate, _ = make_qkv(1, 32, 4, 4, seed=77)
    with pytest.raises(RuntimeError, match="float32"):
        btp_qkv(q.to(DEV), k.to(DEV), v.to(DEV), gate.bfloat16().to(DEV))
    dev = [flat(t).to(DEV) for t in (q, k, v)]
    outs = [torch.empty_like(t) for t in dev]
    dg = torch.empty(1, 32, 4, device=DEV)
    sums = tuple(torch.empty(_btp.mix_backward_sum_rows(1, 32, 4), w, device=DEV) for w in (4, 64, 64))
    with pytest.raises(RuntimeError, match="layer form"):
        _btp.mix_backward(gate.to(DEV), dev[1], dev[0], dev[2], dev[2], dg, outs[1], outs[0], outs[2], 4, 4,
                          sums=sums, qkv_gate=True)
