"""The PyTorch statement of the two-pass algorithm (spear_amd.ops.btp.reference) against the
C oracle: all three decay-matrix constructions, and autograd against the hand-written backward.
The two share no code, so agreement checks both."""

import numpy as np
import pytest
import torch

from oracle import btp_oracle as orc
from spear_amd.ops.btp import reference as ref


def _case(B, H, L, seed, lo=0.05):
    g = torch.Generator().manual_seed(seed)
    a = lo + (1 - lo) * torch.rand(B, H, L, generator=g, dtype=torch.float64)
    x = torch.randn(B, H, 16, L, generator=g, dtype=torch.float64)
    dy = torch.randn(B, H, 16, L, generator=g, dtype=torch.float64)
    return a, x, dy


@pytest.mark.parametrize("ctor", [
    ref.construct_L_ref, ref.construct_L_exp_segsum_log_stable, ref.construct_L_masked_cumprod,
    ref.construct_L_exp_segsum_log, ref.construct_L_cumprod_ratio,
])
def test_decay_matrix_constructors_match_explicit_products(ctor):
    a = 0.2 + 0.8 * torch.rand(3, 16, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    Lm = ctor(a)
    want = torch.zeros(3, 16, 16, dtype=torch.float64)
    for i in range(16):
        for j in range(i + 1):
            want[:, i, j] = a[:, j + 1 : i + 1].prod(-1)
    torch.testing.assert_close(Lm, want, rtol=1e-11, atol=1e-13)


def test_stable_segsum_beats_the_prefix_difference_in_fp32():
    # magnitudes published with the reference (examples/test_stability_log_space.ipynb:258-259):
    # ~1.7e-6 for the prefix-difference form, ~6e-8 for the stable form (fp32, block 16)
    a = torch.rand(512, 16, generator=torch.Generator().manual_seed(2)) * 0.98 + 0.01
    exact = ref.construct_L_ref(a.double())
    err_naive = (ref.construct_L_exp_segsum_log(a).double() - exact).abs().max().item()
    err_stable = (ref.construct_L_exp_segsum_log_stable(a).double() - exact).abs().max().item()
    assert err_stable < 5e-7 and err_stable <= err_naive


@pytest.mark.parametrize("fn", [ref.block_two_pass_ref, ref.block_two_pass_log, ref.block_two_pass_linspace])
@pytest.mark.parametrize("L", [16, 48, 128])
def test_forward_matches_oracle(fn, L):
    a, x, _ = _case(2, 3, L, seed=L)
    np.testing.assert_allclose(fn(a, x, 16).numpy(), orc.forward(a.numpy(), x.numpy()), rtol=1e-10, atol=1e-11)


def test_ref_variant_insists_on_float64():
    a, x, _ = _case(1, 1, 16, seed=0)
    with pytest.raises(AssertionError):
        ref.block_two_pass_ref(a.float(), x.float())


@pytest.mark.parametrize("fn", [ref.block_two_pass_ref, ref.block_two_pass_linspace, ref.block_two_pass_log])
def test_autograd_matches_handwritten_backward(fn):
    a, x, dy = _case(2, 2, 80, seed=5, lo=0.2)
    a.requires_grad_(True)
    x.requires_grad_(True)
    fn(a, x, 16).backward(dy)
    dx, dA = orc.backward(a.detach().numpy(), x.detach().numpy(), dy.numpy())
    np.testing.assert_allclose(x.grad.numpy(), dx, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(a.grad.numpy(), dA, rtol=1e-8, atol=1e-9)


def test_bf16_cpu_path_stays_within_the_reference_forward_limits():
    # limits of the reference's own forward tests (tests/btp/test_numerics.py:27-33)
    from spear_amd.testing.numerics import compute_error_metrics

    g = torch.Generator().manual_seed(123)
    x = torch.randn(2, 8, 16, 512, generator=g).bfloat16()
    a = torch.sigmoid(torch.randn(2, 8, 512, generator=g)).bfloat16()
    got = ref.block_two_pass_log(a.float(), x.float())
    want = torch.from_numpy(orc.forward(a.double().numpy(), x.double().numpy()))
    m = compute_error_metrics(got, want)
    assert m["max_abs"] <= 6e-2 and m["rmse"] <= 1.2e-2 and m["mean_abs"] <= 4e-3


@pytest.mark.parametrize("fn", [ref.block_two_pass_ref, ref.block_two_pass_linspace, ref.block_two_pass_log])
@pytest.mark.parametrize("case", ["smooth", "one_block"])
def test_torch_port_matches_committed_closed_form_vectors(fn, case):
    from helpers import golden_vectors

    v = golden_vectors()[case]
    a, x, dy = (torch.from_numpy(v[n].astype(np.float64)) for n in ("coeff", "x", "dy"))
    a.requires_grad_(True)
    x.requires_grad_(True)
    y = fn(a, x, 16)
    y.backward(dy)
    np.testing.assert_allclose(y.detach().numpy(), v["k2.y"], rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(x.grad.numpy(), v["k2.dx"], rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(a.grad.numpy(), v["k2.dA"], rtol=1e-8, atol=1e-9)


@pytest.mark.parametrize("name", ["log", "linspace"])
def test_cpu_path_matches_vectors_from_the_reference_cpu_path(name):
    """The bfloat16 and float32 CPU paths against outputs of the reference's own functions
    (tests/golden/make_cpu_path_vectors.py). On the machine that wrote the vectors the results are
    bit-identical; the assertion allows one unit in the last place of the dtype, because another CPU's
    matmul kernels may sum in another order."""
    import pathlib

    v = np.load(pathlib.Path(__file__).with_name("golden") / "cpu_path_reference_vectors.npz")
    fn = {"log": ref.block_two_pass_log, "linspace": ref.block_two_pass_linspace}[name]
    a, x = torch.from_numpy(v["a"]).bfloat16(), torch.from_numpy(v["x"]).bfloat16()
    y16 = fn(a, x, 16).float().numpy()
    y32 = fn(a.float(), x.float(), 16).numpy()
    np.testing.assert_allclose(y16, v[f"{name}.bf16"], rtol=2.0 ** -7, atol=2.0 ** -9)
    np.testing.assert_allclose(y32, v[f"{name}.f32"], rtol=2e-6, atol=1e-6)
    y64 = ref.block_two_pass_ref(a.double(), x.double()).numpy()
    np.testing.assert_allclose(y64, v["ref.f64"], rtol=1e-14, atol=1e-15)
