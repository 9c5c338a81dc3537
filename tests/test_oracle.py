"""Pins the CPU oracle (oracle/btp_oracle.c) against things that do not share its code:
the windowed closed form, the token-by-token statement, textbook special cases, finite
differences and the adjoint identity. The reference ships no golden vectors for this path
(its tests compare kernel and Python reference live), so these checks are what anchors parity."""

import numpy as np
import pytest

from oracle import btp_oracle as orc

RNG = np.random.default_rng(20251125)


def rand_case(B, H, L, lo=0.05, hi=1.0):
    a = RNG.uniform(lo, hi, size=(B, H, L))
    x = RNG.standard_normal((B, H, 16, L))
    return a, x


def full_scan(a, x):
    """h_t = a_t h_{t-1} + x_t over the whole sequence (no truncation)."""
    y = np.zeros_like(x)
    h = np.zeros(x.shape[:-1])
    for t in range(x.shape[-1]):
        h = a[..., None, t] * h + x[..., t]
        y[..., t] = h
    return y


@pytest.mark.parametrize("k", [1, 2])
@pytest.mark.parametrize("L", [16, 32, 48, 80])
def test_forward_equals_windowed_closed_form(L, k):
    a, x = rand_case(2, 3, L)
    np.testing.assert_allclose(orc.forward(a, x, k=k), orc.windowed_bruteforce(a, x, k=k), rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("k", [1, 2])
def test_forward_equals_sequential_statement(k):
    a, x = rand_case(2, 2, 160)
    np.testing.assert_allclose(orc.forward(a, x, k=k), orc.forward_sequential(a, x, k=k), rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("L", [16, 32])
def test_short_sequences_are_the_untruncated_scan(L):
    # the window reaches back to the previous block, so up to two blocks nothing is truncated
    a, x = rand_case(1, 2, L)
    np.testing.assert_allclose(orc.forward(a, x, k=2), full_scan(a, x), rtol=1e-12, atol=1e-13)


def test_third_block_does_not_see_the_first():
    a, x = rand_case(1, 1, 48)
    y0 = orc.forward(a, x)
    x2 = x.copy()
    x2[..., :16] += 100.0
    y1 = orc.forward(a, x2)
    assert np.abs(y1[..., :32] - y0[..., :32]).max() > 1.0
    np.testing.assert_array_equal(y1[..., 32:], y0[..., 32:])


def test_k1_is_independent_per_block_scans():
    a, x = rand_case(1, 2, 64)
    y = orc.forward(a, x, k=1)
    for i in range(4):
        s = slice(16 * i, 16 * i + 16)
        np.testing.assert_allclose(y[..., s], full_scan(a[..., s], x[..., s]), rtol=1e-12, atol=1e-13)


def test_unit_decay_is_a_windowed_cumsum():
    _, x = rand_case(1, 1, 64)
    a = np.ones((1, 1, 64))
    y = orc.forward(a, x)
    cs = np.concatenate([np.zeros(x.shape[:-1] + (1,)), np.cumsum(x, -1)], -1)
    for t in range(64):
        w = max(0, (t // 16 - 1) * 16)
        np.testing.assert_allclose(y[..., t], cs[..., t + 1] - cs[..., w], rtol=1e-12, atol=1e-12)


def test_zero_decay_is_identity():
    _, x = rand_case(1, 2, 48)
    np.testing.assert_array_equal(orc.forward(np.zeros((1, 2, 48)), x), x)


def test_constant_decay_of_ones_is_a_geometric_series():
    c, L = 0.7, 64
    a = np.full((1, 1, L), c)
    x = np.ones((1, 1, 16, L))
    y = orc.forward(a, x)
    for t in range(L):
        r, i = t % 16, t // 16
        n_terms = r + 1 + (16 if i > 0 else 0)
        np.testing.assert_allclose(y[0, 0, :, t], (1 - c**n_terms) / (1 - c), rtol=1e-12)


def test_linear_in_x_and_independent_rows():
    a, x1 = rand_case(2, 2, 64)
    _, x2 = rand_case(2, 2, 64)
    lhs = orc.forward(a, 2.0 * x1 - 3.0 * x2)
    np.testing.assert_allclose(lhs, 2.0 * orc.forward(a, x1) - 3.0 * orc.forward(a, x2), rtol=1e-11, atol=1e-11)
    solo = orc.forward(a[1:, :1], x1[1:, :1])
    np.testing.assert_array_equal(solo, orc.forward(a, x1)[1:, :1])


@pytest.mark.parametrize("mode", [orc.L_LOGSUM, orc.L_CUMPROD])
def test_decay_matrix_constructions_agree(mode):
    a, x = rand_case(2, 2, 96, lo=1e-3)
    np.testing.assert_allclose(orc.forward(a, x, l_mode=mode), orc.forward(a, x), rtol=1e-11, atol=1e-12)


def test_checkpoint_is_previous_blocks_local_terminal_state():
    a, x = rand_case(1, 2, 64)
    _, ck = orc.forward(a, x, with_checkpoint=True)
    local = orc.forward(a, x, k=1)
    for i in range(1, 4):
        np.testing.assert_allclose(ck[:, :, i - 1, :], local[..., 16 * i - 1], rtol=1e-12)
    assert np.isnan(ck[:, :, 3, :]).all()  # last slot is never written


@pytest.mark.parametrize("k", [1, 2])
def test_backward_dx_satisfies_the_adjoint_identity(k):
    a, x = rand_case(2, 2, 80)
    dy = RNG.standard_normal(x.shape)
    dx, _ = orc.backward(a, x, dy, k=k)
    assert np.isclose((dy * orc.forward(a, x, k=k)).sum(), (dx * x).sum(), rtol=1e-11)


@pytest.mark.parametrize("k", [1, 2])
def test_backward_matches_central_differences(k):
    a, x = rand_case(1, 2, 64, lo=0.2, hi=0.95)
    dy = RNG.standard_normal(x.shape)
    dx, dA = orc.backward(a, x, dy, k=k)
    loss = lambda aa, xx: (dy * orc.forward(aa, xx, k=k)).sum()
    eps = 1e-6
    for idx in [(0, 0, 0), (0, 0, 15), (0, 1, 16), (0, 1, 17), (0, 0, 31), (0, 1, 32), (0, 0, 47), (0, 1, 63)]:
        ap, am = a.copy(), a.copy()
        ap[idx] += eps
        am[idx] -= eps
        fd = (loss(ap, x) - loss(am, x)) / (2 * eps)
        assert np.isclose(dA[idx], fd, rtol=2e-6, atol=1e-7), (idx, dA[idx], fd)
    for idx in [(0, 0, 3, 0), (0, 1, 7, 15), (0, 0, 0, 16), (0, 1, 15, 40), (0, 0, 9, 63)]:
        xp, xm = x.copy(), x.copy()
        xp[idx] += eps
        xm[idx] -= eps
        fd = (loss(a, xp) - loss(a, xm)) / (2 * eps)
        assert np.isclose(dx[idx], fd, rtol=2e-6, atol=1e-7), (idx, dx[idx], fd)


def test_backward_is_finite_and_right_at_zero_decay():
    # d/da at a == 0 exists (the operator is polynomial in a); formulas that divide by a break here
    a, x = rand_case(1, 1, 48, lo=0.3, hi=0.9)
    a[0, 0, [5, 16, 31, 40]] = 0.0
    dy = RNG.standard_normal(x.shape)
    _, dA = orc.backward(a, x, dy)
    assert np.isfinite(dA).all()
    loss = lambda aa: (dy * orc.forward(aa, x)).sum()
    for t in (5, 16, 31, 40):
        ap, am = a.copy(), a.copy()
        ap[0, 0, t] += 1e-6
        am[0, 0, t] -= 1e-6
        assert np.isclose(dA[0, 0, t], (loss(ap) - loss(am)) / 2e-6, rtol=2e-6, atol=1e-7)


def test_bf16_round_matches_torch():
    torch = pytest.importorskip("torch")
    v = RNG.standard_normal(4096).astype(np.float32) * 3
    v[:4] = [0.0, 1.0, 1.00390625, 3.0e-39]
    ours = orc.bf16_round(v)
    theirs = torch.from_numpy(v).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(ours, theirs)


def test_rejects_bad_arguments():
    a, x = rand_case(1, 1, 24)
    with pytest.raises(ValueError):
        orc.forward(a, x)
    a, x = rand_case(1, 1, 32)
    with pytest.raises(ValueError):
        orc.forward(a, x, k=3)


# ---- committed closed-form vectors -------------------------------------------------------------
@pytest.mark.parametrize("k", [1, 2])
@pytest.mark.parametrize("case", ["smooth", "edges", "one_block"])
def test_oracle_reproduces_committed_closed_form_vectors(case, k):
    from helpers import golden_vectors

    v = golden_vectors()[case]
    a, x, dy = (v[n].astype(np.float64) for n in ("coeff", "x", "dy"))
    for mode in (orc.L_PRODUCT, orc.L_LOGSUM, orc.L_CUMPROD):
        np.testing.assert_allclose(orc.forward(a, x, k=k, l_mode=mode), v[f"k{k}.y"], rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(orc.forward_sequential(a, x, k=k), v[f"k{k}.y"], rtol=1e-11, atol=1e-12)
    dx, dA = orc.backward(a, x, dy, k=k)
    np.testing.assert_allclose(dx, v[f"k{k}.dx"], rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(dA, v[f"k{k}.dA"], rtol=1e-10, atol=1e-11)


def test_oracle_matches_the_reference_float64_path_vectors():
    """The C oracle against the output of the reference's own block_two_pass_ref in float64
    (tests/golden/make_cpu_path_vectors.py)."""
    import pathlib

    v = np.load(pathlib.Path(__file__).with_name("golden") / "cpu_path_reference_vectors.npz")
    a, x = v["a"].astype(np.float64), v["x"].astype(np.float64)
    for mode in (orc.L_PRODUCT, orc.L_LOGSUM, orc.L_CUMPROD):
        np.testing.assert_allclose(orc.forward(a, x, k=2, l_mode=mode), v["ref.f64"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(orc.forward_sequential(a, x, k=2), v["ref.f64"], rtol=1e-12, atol=1e-13)
    dx, dA = orc.backward(a, x, v["dy"].astype(np.float64), k=2)
    np.testing.assert_allclose(dx, v["ref.f64.dx"], rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(dA, v["ref.f64.dA"], rtol=1e-10, atol=1e-11)
