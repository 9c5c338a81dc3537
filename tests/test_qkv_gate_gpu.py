"""The fused kernels in q/k/v/gate terms (SPEAR_MIX_QKV_GATE, ``spear_amd.btp_qkv``):
out = q * btp(exp(gate), k * v) + v on time-major [B, L, H, 16] tensors with an fp32 log-decay gate,
and dq, dk, dv, dgate -- against the float64 composition of the pinned BTP oracle on the same
bf16-rounded inputs. Tolerance: 2e-2 absolute + relative for 16-bit results, and for dgate (fp32 storage,
fp32 arithmetic on bf16 operands) 1e-4 relative to the gradient's scale."""

import numpy as np
import pytest
import torch

from helpers import BF16_ATOL, BF16_RTOL, assert_close, f64
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
    assert_close(f64(flat(dq)), rq, atol * (H // Hkv) ** 0.5, rtol, "dq")
    assert_close(f64(flat(dk)), rk, atol * (H // Hkv) ** 0.5, rtol, "dk")
    scale = max(1.0, float(np.abs(rgate).max()))
    assert float(np.abs(f64(dgate) - rgate).max()) <= 1e-4 * scale, ("dgate", float(np.abs(f64(dgate) - rgate).max()), scale)


@pytest.mark.parametrize("B,L,H,Hkv", [(1, 16, 4, 4), (2, 48, 8, 8), (1, 80, 12, 3), (3, 128, 8, 2), (2, 144, 16, 16),
                                       (1, 512, 32, 32), (1, 1040, 4, 1), (2, 2064, 16, 2), (1, 4096, 8, 8)])
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


def test_benchmark_shape_properties():
    """B=1024, L=128, H=32 (the headline shape in this form): q = 0 returns v, batch rows are independent."""
    from spear_amd import btp_qkv

    q, k, v, gate, _ = make_qkv(1024, 128, 32, 32, seed=75)
    qd, kd, vd, gd = (t.to(DEV) for t in (q, k, v, gate))
    out = btp_qkv(qd, kd, vd, gd)
    assert torch.equal(btp_qkv(torch.zeros_like(qd), kd, vd, gd), vd)     # q = 0 leaves v
    part = btp_qkv(qd[1000:1003].contiguous(), kd[1000:1003].contiguous(), vd[1000:1003].contiguous(), gd[1000:1003].contiguous())
    assert torch.equal(part, out[1000:1003])
    sample = [0, 517, 1023]
    args = [f64(flat(t[sample])) for t in (q, k, v)] + [f64(gate[sample])]
    assert_close(f64(flat(out[sample].cpu())), orc.qkv_gate_forward(*args, 32, 32), BF16_ATOL, BF16_RTOL, "out sample")


def test_rejects_what_it_cannot_do():
    from spear_amd import _btp, btp_qkv

    q, k, v, gate, _ = make_qkv(1, 32, 16, 1, seed=76)
    with pytest.raises(RuntimeError, match="1, 2, 4 or 8"):
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
