"""The fp32 log-space gate entry points (spear_btp_forward_loggate / _backward_loggate, btp_log):
a_t = exp(g_t) is formed in fp32 inside the kernel and the gradient is w.r.t. g_t. The oracle is
the same float64 operator evaluated at a = exp(g) in float64, dgate = a * dA."""

import numpy as np
import pytest
import torch

from helpers import BF16_ATOL, BF16_RTOL, F32_ATOL, F32_RTOL, assert_close, f64
from oracle import btp_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make_log_inputs(B, H, L, seed, kind="softplus", x_std=0.25):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(B, H, 16, L, generator=g) * x_std).bfloat16()
    if kind == "softplus":  # gate = -softplus(N(0,1)), i.e. log sigmoid
        gate = -torch.nn.functional.softplus(torch.randn(B, H, L, generator=g))
    elif kind == "mixed":  # per head: U[-20,-5] (near-total forgetting) or U[-1e-4,0] (near-identity)
        forget = torch.rand(B, H, 1, generator=g) < 0.5
        gate = torch.where(forget, -20.0 + 15.0 * torch.rand(B, H, L, generator=g), -1e-4 * torch.rand(B, H, L, generator=g))
    else:
        raise ValueError(kind)
    dy = torch.randn(B, H, 16, L, generator=g).bfloat16()
    return gate.float().contiguous(), x, dy


def oracle_log(gate, x, dy=None, k=2):
    a = np.exp(f64(gate))
    a[a <= 1e-9] = 0.0
    y = orc.forward(a, f64(x), k=k)
    if dy is None:
        return y
    dx, dA = orc.backward(a, f64(x), f64(dy), k=k)
    return y, dx, dA * a


def run(gate, x, dy, k=2, out_dtype=torch.float32):
    from spear_amd import _btp

    g_, x_, dy_ = gate.to(DEV), x.to(DEV), dy.to(DEV)
    B, H, _, L = x.shape
    y = torch.full((B, H, 16, L), float("nan"), device=DEV, dtype=out_dtype)
    dx = torch.full((B, H, 16, L), float("nan"), device=DEV, dtype=x.dtype)
    dg = torch.full((B, H, L), float("nan"), device=DEV)
    _btp.forward_log(g_, x_, y, k)
    _btp.backward_log(g_, x_, dy_, dx, dg, k)
    torch.cuda.synchronize()
    return y.cpu(), dx.cpu(), dg.cpu()


@pytest.mark.parametrize("k", [2, 1])
@pytest.mark.parametrize("B,H,L", [(1, 1, 16), (2, 3, 48), (1, 2, 128), (2, 2, 144), (2, 8, 512), (1, 2, 1040)])
def test_log_gate_matches_oracle(B, H, L, k):
    gate, x, dy = make_log_inputs(B, H, L, seed=900 + L + k)
    print(f"loggate B={B} H={H} L={L} k={k}", flush=True)
    y, dx, dg = run(gate, x, dy, k=k)
    ry, rdx, rdg = oracle_log(gate, x, dy, k=k)
    assert_close(f64(y), ry, F32_ATOL, F32_RTOL, "y")
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx")
    assert_close(f64(dg), rdg, F32_ATOL, F32_RTOL, "dgate")


def test_log_space_stress_keeps_near_identity_gates():
    # U[-1e-4, 0] gates round to exactly 1.0 as bf16 coefficients; in fp32 log space they survive
    gate, x, dy = make_log_inputs(2, 8, 2048, seed=1236, kind="mixed", x_std=1.0)
    near = gate > -1e-3
    assert (torch.exp(gate)[near].bfloat16() == 1).all() and (torch.exp(gate)[near] < 1).float().mean() > 0.99
    y, dx, dg = run(gate, x, dy)
    ry, rdx, rdg = oracle_log(gate, x, dy)
    assert_close(f64(y), ry, F32_ATOL, F32_RTOL, "y")
    assert_close(f64(dx), rdx, BF16_ATOL, BF16_RTOL, "dx")
    assert_close(f64(dg), rdg, 2e-4, 2e-4, "dgate")


def test_very_negative_gates_are_zero_decay():
    gate, x, dy = make_log_inputs(1, 2, 64, seed=3)
    gate[0, 0, [0, 7, 16, 40]] = -50.0
    gate[0, 1, [31, 32]] = float("-inf")
    y, dx, dg = run(gate, x, dy)
    ry, rdx, rdg = oracle_log(gate, x, dy)
    assert_close(f64(y), ry, F32_ATOL, F32_RTOL, "y")
    assert_close(f64(dg), rdg, F32_ATOL, F32_RTOL, "dgate")
    assert (dg[0, 0, [0, 7, 16, 40]] == 0).all() and (dg[0, 1, [31, 32]] == 0).all()


def test_qkv_gate_composition_through_autograd():
    """The linear-attention reading of the op: x = k*v, y_out = q * btp(exp(gate), x) + v.
    Checks y_out, dq, dk, dv, dgate (fp32 leaves) against the float64 composition."""
    from spear_amd import btp_log

    B, H, L = 2, 4, 256
    g = torch.Generator().manual_seed(77)
    q, k_, v = (0.25 * torch.randn(3, B, H, 16, L, generator=g)).unbind(0)
    gate = -torch.nn.functional.softplus(torch.randn(B, H, L, generator=g))
    dyo = torch.randn(B, H, 16, L, generator=g)

    leaves = [t.clone().to(DEV).requires_grad_(True) for t in (q, k_, v, gate)]
    qd, kd, vd, gd = leaves
    xk = (kd * vd).bfloat16()
    out = qd * btp_log(gd, xk) + vd
    out.backward(dyo.to(DEV))

    # float64 composition; the op sees x and dy rounded to bf16, as on the device
    x_r = (k_ * v).bfloat16()
    h = oracle_log(gate, x_r)
    q64, k64, v64, dyo64 = f64(q), f64(k_), f64(v), f64(dyo)
    dy_op = (dyo * q).float()  # upstream gradient of the op (fp32 on the device)
    _, dx, dgate = oracle_log(gate, x_r, dy_op)
    assert_close(f64(out), q64 * h + v64, 2e-4, 2e-4, "y_out")
    assert_close(f64(qd.grad), dyo64 * h, 2e-4, 2e-4, "dq")
    assert_close(f64(kd.grad), dx * v64, BF16_ATOL, BF16_RTOL, "dk")
    assert_close(f64(vd.grad), dx * k64 + dyo64, BF16_ATOL, BF16_RTOL, "dv")
    assert_close(f64(gd.grad), dgate, 2e-4, 2e-4, "dgate")


def test_log_and_linear_entry_points_agree_on_representable_gates():
    from spear_amd import btp, btp_log

    coeff = torch.sigmoid(torch.randn(2, 4, 128, generator=torch.Generator().manual_seed(5))).bfloat16()
    x = torch.randn(2, 4, 16, 128, generator=torch.Generator().manual_seed(6)).bfloat16()
    y_lin = btp(coeff.to(DEV), x.to(DEV))
    y_log = btp_log(torch.log(coeff.float()).to(DEV), x.to(DEV))
    assert_close(f64(y_log), f64(y_lin), 1e-5, 1e-5, "log vs linear")
