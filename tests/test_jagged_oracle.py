"""Pins oracle/jagged_oracle.py (the float64 restatement of spear/nn/phalanx/inference.py) with facts
that do not come from it: the committed closed-form vectors, a windowed brute-force sum, and the
consistency the streaming form must have with itself (stepping continues a prefill)."""

import numpy as np
import pytest

from helpers import golden_vectors
from oracle import jagged_oracle as jag


def _windowed(a, x, bl, carry_init=None):
    """y_t = sum over s in [start of previous block, t] of (prod_{j=s+1..t} a_j) x_s, plus, in block 0,
    the incoming carry times the gate product from the block start. Plain loops."""
    B, H, D, N = x.shape
    y = np.zeros_like(x)
    for t in range(N):
        blk = t // bl
        for s in range(max(0, (blk - 1) * bl), t + 1):
            y[:, :, :, t] += np.prod(a[:, :, s + 1 : t + 1], axis=-1)[:, :, None] * x[:, :, :, s]
        if blk == 0 and carry_init is not None:
            y[:, :, :, t] += np.prod(a[:, :, 0 : t + 1], axis=-1)[:, :, None] * carry_init
    return y


def _rand(B, H, D, N, seed):
    rng = np.random.RandomState(seed)
    a = 1.0 / (1.0 + np.exp(-rng.randn(B, H, N)))
    return a, rng.randn(B, H, D, N), rng.randn(B, H, D, N), rng.randn(B, H, D, N)


@pytest.mark.parametrize("case", ["smooth", "edges", "one_block"])
def test_sequential_equals_committed_closed_form_vectors(case):
    v = golden_vectors()[case]
    a, x = v["coeff"].astype(np.float64), v["x"].astype(np.float64)
    np.testing.assert_allclose(jag.sequential(x, a, 16), v["k2.y"], rtol=1e-11, atol=1e-12)
    # a block as long as the sequence has no neighbour: the k = 1 vectors of a one-block row
    if case == "one_block":
        np.testing.assert_allclose(jag.sequential(x, a, 16), v["k1.y"], rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("bl,N", [(4, 19), (5, 23), (16, 40), (7, 7), (3, 1)])
def test_sequential_equals_windowed_sum_at_any_block_length(bl, N):
    a, x, _, _ = _rand(2, 2, 3, N, seed=bl * 100 + N)
    np.testing.assert_allclose(jag.sequential(x, a, bl), _windowed(a, x, bl), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(jag.sequential(x, np.log(a), bl, use_log_a=True), _windowed(a, x, bl), rtol=1e-10, atol=1e-11)


def test_carry_init_equals_cutting_a_longer_sequence():
    bl, N = 8, 29
    a, x, _, _ = _rand(1, 2, 4, N, seed=5)
    full = jag.sequential(x, a, bl)
    # terminal local state of block 0 (zero start, 8 steps) is the carry into block 1
    h = np.zeros((1, 2, 4))
    for t in range(bl):
        h = a[:, :, t, None] * h + x[:, :, :, t]
    cut = jag.sequential(x[..., bl:], a[..., bl:], bl, carry_init=h)
    np.testing.assert_allclose(cut, full[..., bl:], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(cut, _windowed(a[..., bl:], x[..., bl:], bl, carry_init=h), rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("log_a", [False, True])
@pytest.mark.parametrize("bl,N", [(4, 13), (16, 50), (5, 5)])
def test_steps_from_the_zero_state_equal_the_sequential_form(bl, N, log_a):
    a, x, c, v = _rand(2, 3, 4, N, seed=N)
    want = jag.sequential(x, a, bl) * c + v
    st = jag.zero_state(2, 3, 4, bl, use_log_r=log_a)
    for t in range(N):
        A_t = np.log(a[:, :, t]) if log_a else a[:, :, t]
        y, new = jag.step(A_t, x[..., t], c[..., t], v[..., t], st, use_log_a=log_a)
        assert new is not st and new.i == (t + 1) % bl
        np.testing.assert_allclose(y, want[..., t], rtol=1e-10, atol=1e-11)
        st = new
    # without C and V the step returns the bare recurrence output
    y, _ = jag.step(a[:, :, 0], x[..., 0], None, None, jag.zero_state(2, 3, 4, bl))
    np.testing.assert_allclose(y, x[..., 0], rtol=0, atol=0)


def test_log_accumulator_clamps_tiny_gates_like_the_reference():
    # a_t below `tiny` enters the log accumulator as log(tiny) (inference.py:205-207) while h uses a_t itself
    st = jag.zero_state(1, 1, 2, 4, use_log_r=True)
    st.c_prev_loc[:] = 3.0
    y, new = jag.step(np.array([[0.0]]), np.ones((1, 1, 2)), None, None, st, tiny=1e-30)
    np.testing.assert_allclose(new.r_pref, np.log(1e-30))
    np.testing.assert_allclose(y, 1.0 + 1e-30 * 3.0)


@pytest.mark.parametrize("bl,L,n", [(16, 37, 30), (16, 8, 9), (4, 6, 11), (5, 3, 1), (16, 17, 16)])
def test_decoding_continues_a_prefill_that_ends_inside_a_block(bl, L, n):
    a, x, c, v = _rand(2, 2, 3, L + n, seed=L * 7 + n)
    Y_all, st_all = jag.prefill(a, x, c, v, block_len=bl)
    np.testing.assert_allclose(Y_all, jag.sequential(x, a, bl) * c + v, rtol=0, atol=0)
    Y, st = jag.prefill(a[..., :L], x[..., :L], c[..., :L], v[..., :L], block_len=bl)
    np.testing.assert_allclose(Y, Y_all[..., :L], rtol=1e-12, atol=1e-13)
    assert st.i == L % bl and not st.use_log_r
    for t in range(L, L + n):
        y, st = jag.step(a[:, :, t], x[..., t], c[..., t], v[..., t], st)
        np.testing.assert_allclose(y, Y_all[..., t], rtol=1e-10, atol=1e-11)
    # and the state reached by stepping is the state a longer prefill hands over
    if (L + n) % bl != 0:
        for got, want in ((st.h_loc, st_all.h_loc), (st.r_pref, st_all.r_pref), (st.c_prev_loc, st_all.c_prev_loc)):
            np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-11)
        assert st.i == st_all.i


def test_prefill_state_after_a_full_block_follows_the_reference_text():
    # inference.py:327-341: carry snapshot taken and gate product reset, but h_loc keeps the block's
    # terminal local state; a step from that state therefore counts it twice. (The same case against
    # the reference's own output: test_oracle_reproduces_the_reference_vectors[full].)
    bl, L = 4, 8
    a, x, c, v = _rand(1, 2, 3, L + 1, seed=3)
    _, st = jag.prefill(a[..., :L], x[..., :L], c[..., :L], v[..., :L], block_len=bl)
    h_last = np.zeros((1, 2, 3))
    for t in range(L - bl, L):
        h_last = a[:, :, t, None] * h_last + x[:, :, :, t]
    assert st.i == 0
    np.testing.assert_allclose(st.h_loc, h_last, rtol=1e-13)
    np.testing.assert_allclose(st.c_prev_loc, h_last, rtol=1e-13)
    np.testing.assert_allclose(st.r_pref, 1.0)
    y, _ = jag.step(a[:, :, L], x[..., L], c[..., L], v[..., L], st)
    np.testing.assert_allclose(y, (x[..., L] + 2 * a[:, :, L, None] * h_last) * c[..., L] + v[..., L], rtol=1e-12)


# ---- vectors from the reference's own functions ------------------------------------------------------
@pytest.mark.parametrize("case", ["full", "ragged", "short", "one_block", "bl4"])
def test_oracle_reproduces_the_reference_vectors(case):
    """Prefill output, hand-over state (also after a full last block, the case no identity pins) and the
    decode steps taken from that state, against vectors computed by the reference's parallel_jagged /
    step_jagged in float64 (tests/golden/make_jagged_vectors.py)."""
    from helpers import jagged_reference_vectors

    v = jagged_reference_vectors()[case]
    L, bl, steps, i_ref = (int(t) for t in v["meta"])
    A, X, C, V = (v[n].astype(np.float64) for n in "AXCV")
    Y, st = jag.prefill(A[..., :L], X[..., :L], C[..., :L], V[..., :L], block_len=bl)
    np.testing.assert_allclose(Y, v["Y"], rtol=1e-12, atol=1e-13)
    assert st.i == i_ref
    np.testing.assert_allclose(st.h_loc, v["h_loc"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(st.r_pref, v["r_pref"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(st.c_prev_loc, v["c_prev_loc"], rtol=1e-12, atol=1e-13)
    for k in range(steps):
        t = L + k
        y, st = jag.step(A[:, :, t], X[..., t], C[..., t], V[..., t], st)
        np.testing.assert_allclose(y, v["y_steps"][..., k], rtol=1e-11, atol=1e-12)
    final = np.concatenate([st.h_loc.ravel(), st.r_pref.ravel(), st.c_prev_loc.ravel(), [st.i]])
    np.testing.assert_allclose(final, v["final"], rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("H,Hkv,L", [(4, 4, 40), (8, 2, 33), (12, 3, 64)])
def test_layer_steps_equal_the_two_pass_statement_of_the_stage(H, Hkv, L):
    """Stepping the layer-layout token update through a sequence gives what the two-pass (block) statement of
    the same stage gives for the whole sequence: the gates, the kv-head sharing and the layout of layer_step
    are pinned by an algorithm that shares none of its code."""
    from oracle import btp_oracle as orc

    rng = np.random.default_rng(H * 100 + L)
    B = 2
    Lp = -(-L // 16) * 16  # the block statement needs whole blocks; the extra steps do not touch earlier outputs
    a = rng.normal(size=(B, Lp, H))
    b = rng.normal(size=(B, Lp, Hkv * 16))
    c = rng.normal(size=(B, Lp, Hkv * 16))
    v = rng.normal(size=(B, Lp, H * 16))
    want = orc.phalanx_mix_forward(a, b, c, v, H, Hkv)
    state = jag.zero_state(B, H, 16, 16)
    for t in range(L):
        out, state = jag.layer_step(a[:, t], b[:, t], c[:, t], v[:, t], state, H, Hkv)
        np.testing.assert_allclose(out, want[:, t], rtol=1e-10, atol=1e-10)
    assert state.i == L % 16
