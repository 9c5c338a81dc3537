"""float64 numpy restatement of the reference's streaming (token-by-token) form of the operator.

TEST INFRASTRUCTURE ONLY: imported by tests/ and by ``__graft_entry__.smoke``; the shipped package
never imports it.

What follows what (paths relative to the reference repository):
    sequential()  spear/nn/phalanx/inference.py:36-92    jagged_band_infer_sequential
    step()        spear/nn/phalanx/inference.py:178-278  step_jagged (also JaggedBandState.step, :121-140,
                                                          which is the same update without ``* C + V``)
    prefill()     spear/nn/phalanx/inference.py:281-360  parallel_jagged: outputs and the hand-over state
    layer_step()  spear/nn/phalanx/swr.py:196-221 (the layer's gates and kv-head expansion) feeding step()

How each is pinned (tests/test_jagged_oracle.py); none of the tests imports the reference:
    sequential    equals the committed closed-form vectors at block length 16 and a windowed brute-force
                  sum at other block lengths; carry_init equals cutting a longer sequence
    step          N steps from the zero state equal sequential() * C + V across block boundaries, in
                  linear and in log-r mode
    prefill       Y equals sequential() * C + V; the state is pinned by continuing: prefill(L) followed
                  by steps equals prefill(L + n) whenever L is not a multiple of the block length.
                  When L IS a multiple of the block length the reference hands over h_loc = the last
                  block's terminal local state instead of zero (inference.py:327-341), which no
                  identity fixes (stepping from it counts that state twice); that case, like the others,
                  is pinned by vectors computed with the reference's own parallel_jagged / step_jagged
                  (tests/golden/make_jagged_vectors.py -> jagged_reference_vectors.npz).
    layer_step    L steps from the zero state equal the two-pass statement of the same stage on the whole
                  sequence (oracle.btp_oracle.phalanx_mix_forward, itself pinned), with shared kv heads
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np

F32_TINY = float(np.finfo(np.float32).tiny)


@dataclass
class State:
    """Fields of the reference's JagState (inference.py:142-165) as float64 arrays."""

    h_loc: np.ndarray        # [B, H, D]
    r_pref: np.ndarray       # [B, H]; holds log(r) when use_log_r
    c_prev_loc: np.ndarray   # [B, H, D]
    i: int
    block_len: int
    use_log_r: bool = False


def zero_state(B: int, H: int, D: int, block_len: int, use_log_r: bool = False) -> State:
    r = np.zeros((B, H)) if use_log_r else np.ones((B, H))
    return State(np.zeros((B, H, D)), r, np.zeros((B, H, D)), 0, block_len, use_log_r)


def sequential(u, a, block_len: int, *, use_log_a: bool = False, carry_init=None) -> np.ndarray:
    """u [B,H,D,N], a [B,H,N] -> y [B,H,D,N]: block-local scan from zero plus the frozen terminal
    local state of the previous block times the inclusive in-block gate product."""
    u = np.asarray(u, dtype=np.float64)
    g = np.exp(np.asarray(a, dtype=np.float64)) if use_log_a else np.asarray(a, dtype=np.float64)
    B, H, D, N = u.shape
    y = np.empty_like(u)
    c_prev = np.zeros((B, H, D)) if carry_init is None else np.array(carry_init, dtype=np.float64)
    y_loc = np.zeros((B, H, D))
    r = np.ones((B, H, 1))
    i = 0
    for t in range(N):
        a_t = g[:, :, t, None]
        y_loc = a_t * y_loc + u[:, :, :, t]
        r = a_t * r
        y[:, :, :, t] = y_loc + r * c_prev
        i += 1
        if i == block_len:
            c_prev = y_loc.copy()
            y_loc = np.zeros((B, H, D))
            r = np.ones((B, H, 1))
            i = 0
    return y


def step(A_t, X_t, C_t, V_t, state: State, *, use_log_a: bool = False, tiny: float = F32_TINY):
    """One token. A_t [B,H] (a_t, or log a_t with use_log_a), X_t/C_t/V_t [B,H,D] (C_t, V_t may be
    None: then y is returned without ``* C + V``). Returns (y_t, new State); `state` is not modified."""
    A_t = np.asarray(A_t, dtype=np.float64)
    a = np.exp(A_t) if use_log_a else A_t
    h = a[..., None] * state.h_loc + np.asarray(X_t, dtype=np.float64)
    log_mode = state.use_log_r or use_log_a
    if log_mode:
        prev = state.r_pref if state.use_log_r else np.zeros_like(a)  # a fresh log accumulator starts at log 1
        log_r = prev + np.log(np.maximum(a, tiny))
        r = np.exp(log_r)
    else:
        r = a * state.r_pref
    y = h + r[..., None] * state.c_prev_loc
    if C_t is not None:
        y = y * np.asarray(C_t, dtype=np.float64) + np.asarray(V_t, dtype=np.float64)
    if state.i + 1 == state.block_len:
        r_new = np.zeros_like(a) if log_mode else np.ones_like(a)
        return y, State(np.zeros_like(h), r_new, h.copy(), 0, state.block_len, log_mode)
    return y, State(h, log_r if log_mode else r, state.c_prev_loc, state.i + 1, state.block_len, log_mode)


def prefill(A, X, C, V, *, block_len: int, use_log_a: bool = False):
    """A [B,H,L], X/C/V [B,H,D,L] -> (Y [B,H,D,L], State after the last token)."""
    X = np.asarray(X, dtype=np.float64)
    a = np.exp(np.asarray(A, dtype=np.float64)) if use_log_a else np.asarray(A, dtype=np.float64)
    B, H, D, L = X.shape
    Y = sequential(X, a, block_len) * np.asarray(C, dtype=np.float64) + np.asarray(V, dtype=np.float64)

    def local_at(t):  # block-local state and inclusive gate product at step t
        s = (t // block_len) * block_len
        h = np.zeros((B, H, D))
        r = np.ones((B, H))
        for q in range(s, t + 1):
            h = a[:, :, q, None] * h + X[:, :, :, q]
            r = r * a[:, :, q]
        return h, r

    h_tail, r_tail = local_at(L - 1)
    if (L - 1) % block_len == block_len - 1:
        # full last block: carry snapshot taken, gate product reset, h_loc NOT reset (see module docstring)
        return Y, State(h_tail, np.ones((B, H)), h_tail.copy(), 0, block_len)
    done = L // block_len
    c_prev = local_at(done * block_len - 1)[0] if done > 0 else np.zeros((B, H, D))
    return Y, State(h_tail, r_tail, c_prev, (L - 1) % block_len + 1, block_len)


def layer_step(a_logit, b_logit, c, v, state: State, heads: int, kv_heads: int | None = None):
    """One token of the Phalanx mixing stage on the projections' outputs for that token: a_logit [B, H],
    b_logit / c [B, kv_heads * D], v [B, H * D]. The gates and the kv-head expansion are the layer's
    (swr.py:196-221: A = sigmoid(a), X = sigmoid(b) * v, head h uses b / c of kv head h // (H // kv_heads)), the
    update is step(). Returns (out [B, H * D], new State)."""
    kv = heads if kv_heads is None else kv_heads
    a64, b64, c64, v64 = (np.asarray(t, dtype=np.float64) for t in (a_logit, b_logit, c, v))
    B = v64.shape[0]
    D = v64.shape[1] // heads
    sig = lambda z: 1.0 / (1.0 + np.exp(-z))
    V = v64.reshape(B, heads, D)
    G = np.repeat(sig(b64).reshape(B, kv, D), heads // kv, axis=1)
    C = np.repeat(c64.reshape(B, kv, D), heads // kv, axis=1)
    y, new = step(sig(a64), G * V, C, V, state)
    return y.reshape(B, heads * D), new
