"""Parity of the streaming kernels (prefill with state hand-over, decode step), called through
spear_amd.nn.phalanx.inference and the C ABI beneath it, with the float64 oracle
(oracle/jagged_oracle.py) on the same rounded inputs.

Tolerances: 16-bit tensors within 2e-2 (absolute + relative), fp32 tensors within 1e-4."""

import numpy as np
import pytest
import torch

from helpers import BF16_ATOL, BF16_RTOL, F32_ATOL, F32_RTOL, assert_close, f64
from oracle import jagged_oracle as jag

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def make(B, H, D, L, seed, dtype=torch.bfloat16, a_dtype=None, log_a=False):
    g = torch.Generator(device="cpu").manual_seed(seed)
    gate = -torch.nn.functional.softplus(torch.randn(B, H, L, generator=g))  # log sigmoid(N(0,1))
    A = (gate if log_a else gate.exp()).to(dtype if a_dtype is None else a_dtype)
    X = (0.5 * torch.randn(B, H, D, L, generator=g)).to(dtype)
    C = torch.randn(B, H, D, L, generator=g).to(dtype)
    V = torch.randn(B, H, D, L, generator=g).to(dtype)
    return A, X, C, V


def tol(dtype):
    return (F32_ATOL, F32_RTOL) if dtype == torch.float32 else (BF16_ATOL, BF16_RTOL)


def check_state(st, ref, atol, rtol, what):
    assert st.i == ref.i and st.block_len == ref.block_len, what
    assert_close(f64(st.h_loc), ref.h_loc, atol, rtol, f"{what} h_loc")
    assert_close(f64(st.c_prev_loc), ref.c_prev_loc, atol, rtol, f"{what} c_prev_loc")
    r = st.log_r_pref if st.use_log_r else st.r_pref
    assert_close(f64(r), ref.r_pref, atol, rtol, f"{what} r")


TILED = [(2, 3, 16), (1, 2, 24), (2, 2, 40), (1, 4, 128), (2, 2, 136), (1, 2, 264), (1, 3, 1032), (2, 2, 2048), (3, 1, 8)]


@pytest.mark.parametrize("state_dtype", [None, torch.float32], ids=["state16", "state32"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("B,H,L", TILED)
def test_prefill_16bit_matches_oracle(B, H, L, dtype, state_dtype):
    from spear_amd.nn.phalanx.inference import parallel_jagged

    A, X, C, V = make(B, H, 16, L, seed=L + B, dtype=dtype)
    print(f"prefill tiled B={B} H={H} L={L} {dtype} state={state_dtype}", flush=True)
    Y, st = parallel_jagged(A.to(DEV), X.to(DEV), C.to(DEV), V.to(DEV), block_len=16, state_dtype=state_dtype)
    rY, rst = jag.prefill(f64(A), f64(X), f64(C), f64(V), block_len=16)
    assert Y.dtype == dtype and st.h_loc.dtype == (state_dtype or dtype)
    assert_close(f64(Y), rY, BF16_ATOL, BF16_RTOL, "Y")
    check_state(st, rst, BF16_ATOL, BF16_RTOL, "state")
    if state_dtype == torch.float32:  # fp32 state of the fp32 arithmetic: tight
        check_state(st, rst, F32_ATOL, F32_RTOL, "state fp32")


@pytest.mark.parametrize("B,H,L", [(2, 2, 48), (1, 3, 200), (1, 2, 1160)])
def test_prefill_fp32_log_gate_matches_oracle(B, H, L):
    from spear_amd.nn.phalanx.inference import parallel_jagged

    A, X, C, V = make(B, H, 16, L, seed=9 + L, a_dtype=torch.float32, log_a=True)
    print(f"prefill tiled log B={B} H={H} L={L}", flush=True)
    Y, st = parallel_jagged(A.to(DEV), X.to(DEV), C.to(DEV), V.to(DEV), block_len=16, use_log_a=True)
    rY, rst = jag.prefill(f64(A), f64(X), f64(C), f64(V), block_len=16, use_log_a=True)
    assert st.r_pref.dtype == torch.float32 and st.h_loc.dtype == torch.bfloat16
    assert_close(f64(Y), rY, BF16_ATOL, BF16_RTOL, "Y")
    check_state(st, rst, BF16_ATOL, BF16_RTOL, "state")


ANY = [  # B, H, D, L, block_len, dtype, a_dtype, log_a
    (2, 2, 16, 37, 16, torch.bfloat16, None, False),      # odd length: rows lose 16-byte alignment
    (1, 3, 16, 5, 16, torch.bfloat16, None, False),       # shorter than a block
    (2, 1, 16, 1, 16, torch.float16, None, False),
    (1, 2, 16, 64, 16, torch.float32, None, False),       # fp32 tensors
    (2, 2, 16, 50, 16, torch.float32, None, True),
    (1, 2, 16, 48, 16, torch.bfloat16, None, True),       # 16-bit log gate
    (2, 2, 16, 203, 16, torch.float16, None, True),       # 16-bit log gate, odd length, two spans
    (1, 2, 16, 48, 16, torch.bfloat16, torch.float32, False),  # fp32 linear gate with 16-bit tensors
    (2, 3, 8, 45, 4, torch.bfloat16, None, False),        # other block length and head size
    (1, 2, 3, 23, 5, torch.float32, None, False),
    (1, 1, 24, 33, 7, torch.float16, None, False),
]


@pytest.mark.parametrize("B,H,D,L,bl,dtype,a_dtype,log_a", ANY)
def test_prefill_general_shapes_and_dtypes_match_oracle(B, H, D, L, bl, dtype, a_dtype, log_a):
    from spear_amd.nn.phalanx.inference import parallel_jagged

    A, X, C, V = make(B, H, D, L, seed=L * 3 + D, dtype=dtype, a_dtype=a_dtype, log_a=log_a)
    print(f"prefill any B={B} H={H} D={D} L={L} bl={bl} {dtype} a={a_dtype} log={log_a}", flush=True)
    Y, st = parallel_jagged(A.to(DEV), X.to(DEV), C.to(DEV), V.to(DEV), block_len=bl, use_log_a=log_a)
    rY, rst = jag.prefill(f64(A), f64(X), f64(C), f64(V), block_len=bl, use_log_a=log_a)
    assert_close(f64(Y), rY, *tol(dtype), "Y")
    check_state(st, rst, *tol(dtype), "state")


@pytest.mark.parametrize("B,H,D,N,bl,dtype", [(2, 2, 16, 160, 16, torch.bfloat16), (1, 2, 16, 45, 16, torch.bfloat16),
                                              (1, 3, 16, 96, 16, torch.float32), (2, 2, 4, 30, 6, torch.float32)])
@pytest.mark.parametrize("with_carry", [False, True])
def test_sequential_form_matches_oracle(B, H, D, N, bl, dtype, with_carry):
    from spear_amd.nn.phalanx.inference import jagged_band_infer_sequential

    A, X, _, _ = make(B, H, D, N, seed=N + bl, dtype=dtype)
    carry = torch.randn(B, H, D, generator=torch.Generator().manual_seed(N)).to(dtype) if with_carry else None
    print(f"sequential B={B} H={H} D={D} N={N} bl={bl} {dtype} carry={with_carry}", flush=True)
    y = jagged_band_infer_sequential(X.to(DEV), A.to(DEV), bl, carry_init=None if carry is None else carry.to(DEV))
    want = jag.sequential(f64(X), f64(A), bl, carry_init=None if carry is None else f64(carry))
    assert y.dtype == dtype and y.shape == X.shape
    assert_close(f64(y), want, *tol(dtype), "y")


STEP = [  # B, H, D, block_len, dtype, state_dtype, log_a
    (2, 3, 16, 16, torch.bfloat16, torch.float32, False),
    (2, 3, 16, 16, torch.bfloat16, torch.float32, True),
    (1, 4, 16, 16, torch.float16, torch.float32, False),
    (2, 2, 16, 16, torch.float32, torch.float32, False),
    (2, 2, 16, 16, torch.float32, torch.float32, True),
    (3, 2, 64, 4, torch.float32, torch.float32, False),   # 8 octets per head
    (2, 2, 24, 5, torch.float32, torch.float32, False),   # 3 octets per head: per-head kernel
    (2, 5, 3, 6, torch.bfloat16, torch.float32, False),   # odd head size: per-head kernel
]


@pytest.mark.parametrize("inplace", [False, True])
@pytest.mark.parametrize("B,H,D,bl,dtype,state_dtype,log_a", STEP)
def test_decode_steps_match_oracle_across_block_boundaries(B, H, D, bl, dtype, state_dtype, log_a, inplace):
    from spear_amd.nn.phalanx.inference import JagState, step_jagged

    N = 2 * bl + 3
    A, X, C, V = make(B, H, D, N, seed=bl + D, dtype=dtype, a_dtype=torch.float32, log_a=log_a)  # fp32 gate: fp32 r
    print(f"steps B={B} H={H} D={D} bl={bl} {dtype} log={log_a} inplace={inplace}", flush=True)
    st = JagState(torch.zeros(B, H, D, device=DEV, dtype=state_dtype), None,
                  torch.zeros(B, H, D, device=DEV, dtype=state_dtype), 0, bl)
    ref = jag.zero_state(B, H, D, bl)
    Ad, Xd, Cd, Vd = (t.to(DEV) for t in (A, X, C, V))
    atol, rtol = tol(dtype)
    for t in range(N):
        before = st.clone_detached()
        y, new = step_jagged(Ad[:, :, t], Xd[..., t], Cd[..., t], Vd[..., t], st, use_log_a=log_a, inplace=inplace)
        ry, ref = jag.step(f64(A[:, :, t]), f64(X[..., t]), f64(C[..., t]), f64(V[..., t]), ref, use_log_a=log_a)
        assert y.dtype == dtype
        assert_close(f64(y), ry, atol, rtol, f"y at token {t}")
        assert (new is st) == inplace and new.use_log_r == log_a
        if not inplace:  # the old state is untouched, as in the reference
            assert torch.equal(st.h_loc, before.h_loc) and torch.equal(st.c_prev_loc, before.c_prev_loc)
        check_state(new, ref, atol, rtol, f"state after token {t}")
        st = new


def test_decode_with_16bit_state_stays_within_tolerance_of_oracle():
    from spear_amd.nn.phalanx.inference import JagState, step_jagged

    B, H, D, bl, N = 2, 4, 16, 16, 40
    A, X, C, V = make(B, H, D, N, seed=77)
    st = JagState(torch.zeros(B, H, D, device=DEV, dtype=torch.bfloat16), None,
                  torch.zeros(B, H, D, device=DEV, dtype=torch.bfloat16), 0, bl)
    ref = jag.zero_state(B, H, D, bl)
    for t in range(N):
        y, st = step_jagged(A[:, :, t].to(DEV), X[..., t].to(DEV), C[..., t].to(DEV), V[..., t].to(DEV), st)
        ry, ref = jag.step(f64(A[:, :, t]), f64(X[..., t]), f64(C[..., t]), f64(V[..., t]), ref)
        # the state is rounded to bf16 after every token: errors add up inside a block
        assert_close(f64(y), ry, 6e-2, 4e-2, f"y at token {t}")
    assert st.r_pref.dtype == torch.bfloat16 and st.h_loc.dtype == torch.bfloat16


@pytest.mark.parametrize("L,n", [(40, 30), (8, 9), (17, 16), (129, 5)])
def test_decoding_continues_the_prefill(L, n):
    from spear_amd.nn.phalanx.inference import parallel_jagged, step_jagged

    B, H = 2, 3
    A, X, C, V = make(B, H, 16, L + n, seed=L + n)
    Ad, Xd, Cd, Vd = (t.to(DEV) for t in (A, X, C, V))
    rY, _ = jag.prefill(f64(A), f64(X), f64(C), f64(V), block_len=16)
    Y, st = parallel_jagged(Ad[..., :L].contiguous(), Xd[..., :L].contiguous(), Cd[..., :L].contiguous(),
                            Vd[..., :L].contiguous(), block_len=16, state_dtype=torch.float32)
    assert_close(f64(Y), rY[..., :L], BF16_ATOL, BF16_RTOL, "prefill part")
    for t in range(L, L + n):
        y, st = step_jagged(Ad[:, :, t], Xd[..., t], Cd[..., t], Vd[..., t], st, inplace=True)
        assert_close(f64(y), rY[..., t], BF16_ATOL, BF16_RTOL, f"decode token {t}")


def test_band_state_class_matches_sequential_form():
    from spear_amd.nn.phalanx.inference import JaggedBandState

    B, H, D, bl, N = 2, 2, 16, 16, 37
    A, X, _, _ = make(B, H, D, N, seed=4, dtype=torch.float32)
    want = jag.sequential(f64(X), f64(A), bl)
    st = JaggedBandState(B, H, D, bl, device=DEV, dtype=torch.float32)
    for t in range(N):
        a_t = A[:, :, t].to(DEV)
        y = st.step(a_t.unsqueeze(-1) if t % 2 else a_t, X[..., t].to(DEV))
        assert_close(f64(y), want[..., t], F32_ATOL, F32_RTOL, f"token {t}")
    assert st.i == N % bl and st.r_pref.shape == (B, H, 1)
    st.reset_block()
    assert st.i == 0 and float(st.y_loc.abs().max()) == 0.0
    # log-space gates: same outputs
    st = JaggedBandState(B, H, D, bl, device=DEV, dtype=torch.float32)
    for t in range(bl + 2):
        y = st.step(A[:, :, t].log().to(DEV), X[..., t].to(DEV), use_log_a=True)
        assert_close(f64(y), want[..., t], F32_ATOL, F32_RTOL, f"log token {t}")


def test_prefill_agrees_with_the_training_kernel_at_benchmark_size():
    """Size-independent property at the benchmark shape (B=1024 would take the oracle minutes): the
    prefill output equals the stand-alone forward kernel's y * C + V, and its hand-over carry lets
    the sequential form continue a row cut at a block boundary."""
    from spear_amd import btp
    from spear_amd.nn.phalanx.inference import jagged_band_infer_sequential, parallel_jagged

    B, H, L = 256, 32, 128
    g = torch.Generator(device="cpu").manual_seed(1234)
    A = torch.sigmoid(torch.randn(B, H, L, generator=g)).bfloat16().to(DEV)
    X = (0.25 * torch.randn(B, H, 16, L, generator=g)).bfloat16().to(DEV)
    C = torch.randn(B, H, 16, L, generator=g).bfloat16().to(DEV)
    V = torch.randn(B, H, 16, L, generator=g).bfloat16().to(DEV)
    Y, st = parallel_jagged(A, X, C, V, block_len=16, state_dtype=torch.float32)
    y32 = btp(A, X, output_dtype=torch.float32)
    want = y32 * C.float() + V.float()
    err = (Y.float() - want).abs() - (BF16_ATOL / 4 + BF16_RTOL / 4 * want.abs())  # only output rounding differs
    assert float(err.max()) <= 0, float(err.max())
    cut = 64
    Yc, stc = parallel_jagged(A[..., :cut].contiguous(), X[..., :cut].contiguous(), C[..., :cut].contiguous(),
                              V[..., :cut].contiguous(), block_len=16, state_dtype=torch.float32)
    rest = jagged_band_infer_sequential(X[..., cut:].contiguous().float(), A[..., cut:].contiguous().float(), 16,
                                        carry_init=stc.c_prev_loc)
    assert float((rest - y32[..., cut:]).abs().max()) <= 1e-4 * (1 + float(y32.abs().max()))
    assert torch.equal(Yc, Y[..., :cut])


def test_streaming_functions_reject_cpu_tensors_and_bad_arguments():
    from spear_amd import _btp
    from spear_amd.nn.phalanx.inference import JaggedBandState, jagged_band_infer_sequential, parallel_jagged

    A, X, C, V = make(1, 2, 16, 32, seed=0)
    with pytest.raises(RuntimeError, match="must be on a GPU"):
        parallel_jagged(A, X, C, V, block_len=16)
    with pytest.raises(RuntimeError, match="must be on a GPU"):
        jagged_band_infer_sequential(X, A, 16)
    with pytest.raises(RuntimeError, match="must be a GPU"):
        JaggedBandState(1, 2, 16, 16, device="cpu")
    Ad, Xd, Cd, Vd = (t.to(DEV) for t in (A, X, C, V))
    with pytest.raises(RuntimeError, match="given together"):
        _btp.jagged_prefill(Ad, Xd, Cd, None, None, torch.empty_like(Xd), None, None, None, 16, False)
    with pytest.raises(RuntimeError, match="shape"):
        _btp.jagged_prefill(Ad[..., :16].contiguous(), Xd, None, None, None, torch.empty_like(Xd), None, None, None, 16, False)
    with pytest.raises(RuntimeError, match="float32 or match"):
        _btp.jagged_prefill(Ad.half(), Xd, None, None, None, torch.empty_like(Xd), None, None, None, 16, False)


def test_one_block_period_of_decode_steps_replays_as_a_hip_graph():
    """The step entry point allocates nothing and takes the block boundary as an argument, so the 16
    steps of one block period, updating the state in place, form a graph that can be replayed for
    every following period. Each replay (with eager work and synchronisation in between) is checked
    against the oracle continuing from the same state."""
    from spear_amd import _btp

    B, H, D, bl = 3, 4, 16, 16
    A, X, C, V = make(B, H, D, 4 * bl, seed=31, a_dtype=torch.float32)
    rY, _ = jag.prefill(f64(A), f64(X), f64(C), f64(V), block_len=bl)
    # static input buffers, [token][...] so that every captured launch reads a fixed address
    a_buf = torch.empty(bl, B, H, device=DEV)
    x_buf, c_buf, v_buf, y_buf = (torch.empty(bl, B, H, D, device=DEV, dtype=torch.bfloat16) for _ in range(4))
    h = torch.zeros(B, H, D, device=DEV)
    cp = torch.zeros(B, H, D, device=DEV)
    r = torch.ones(B, H, device=DEV)

    def period():
        for i in range(bl):
            _btp.jagged_step(a_buf[i], x_buf[i], c_buf[i], v_buf[i], y_buf[i], h, r, cp, h, r, cp,
                             i == bl - 1, False, False, 0.0)

    def load(p):  # eager copies between replays
        sl = slice(p * bl, (p + 1) * bl)
        a_buf.copy_(A[..., sl].permute(2, 0, 1))
        for buf, src in ((x_buf, X), (c_buf, C), (v_buf, V)):
            buf.copy_(src[..., sl].permute(3, 0, 1, 2))

    load(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        period()  # warm-up on a side stream; its state update is undone below
    torch.cuda.current_stream().wait_stream(side)
    h.zero_(); cp.zero_(); r.fill_(1.0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        period()
    h.zero_(); cp.zero_(); r.fill_(1.0)  # capture does not run the kernels, but be explicit
    for p in range(4):
        load(p)
        y_buf.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = f64(y_buf).transpose(1, 2, 3, 0)  # [B, H, D, token]
        assert_close(got, rY[..., p * bl:(p + 1) * bl], BF16_ATOL, BF16_RTOL, f"period {p}")


@pytest.mark.parametrize("offset", [0, 1, 2, 3], ids=lambda o: f"off{o}")
@pytest.mark.parametrize("L", [1, 2, 3, 7, 9, 15, 17, 31, 33, 126, 127, 129, 130, 255, 257, 1037])
def test_prefill_rows_of_any_length_and_alignment(L, offset):
    """Prompt lengths that are not a multiple of 8 and tensors that start on any 2-byte boundary: the
    tiled kernel realigns rows in registers. Output and state against the oracle, and the elements
    around the output tensor must stay untouched."""
    from spear_amd import _btp

    B, H, D = 2, 3, 16
    A, X, C, V = make(B, H, D, L, seed=7000 + L)

    def shifted(t):  # the same values in a buffer that starts `offset` elements into an allocation
        buf = torch.full((t.numel() + 16,), float("nan"), dtype=t.dtype, device=DEV)
        view = buf[offset:offset + t.numel()].view(t.shape)
        view.copy_(t)
        return buf, view

    (_, a), (_, x), (_, c), (_, v) = (shifted(t) for t in (A, X, C, V))
    ybuf, y = shifted(torch.full(X.shape, float("nan"), dtype=X.dtype))
    h, cp = (torch.full((B, H, D), float("nan"), device=DEV) for _ in range(2))
    r = torch.full((B, H), float("nan"), device=DEV)
    print(f"ragged prefill L={L} offset={offset}", flush=True)
    _btp.jagged_prefill(a, x, c, v, None, y, h, r, cp, 16, False)
    torch.cuda.synchronize()
    rY, rst = jag.prefill(f64(A), f64(X), f64(C), f64(V), block_len=16)
    assert_close(f64(y), rY, BF16_ATOL, BF16_RTOL, "Y")
    assert_close(f64(h), rst.h_loc, F32_ATOL, F32_RTOL, "h_loc")
    assert_close(f64(cp), rst.c_prev_loc, F32_ATOL, F32_RTOL, "c_prev_loc")
    assert_close(f64(r), rst.r_pref, F32_ATOL, F32_RTOL, "r_pref")
    guard = torch.cat([ybuf[:offset], ybuf[offset + X.numel():]])
    assert bool(torch.isnan(guard).all()), "elements outside the output tensor were written"


@pytest.mark.parametrize("case", ["full", "ragged", "short", "one_block", "bl4"])
def test_kernels_match_the_reference_vectors(case):
    """The HIP prefill and decode kernels against vectors computed by the reference's own
    parallel_jagged / step_jagged (tests/golden/make_jagged_vectors.py), including the state handed
    over after a full last block and the steps taken from it."""
    from helpers import jagged_reference_vectors
    from spear_amd.nn.phalanx.inference import parallel_jagged, step_jagged

    v = jagged_reference_vectors()[case]
    L, bl, steps, i_ref = (int(t) for t in v["meta"])
    A, X, C, V = (torch.from_numpy(v[n]).bfloat16().to(DEV) for n in "AXCV")
    for n, t in zip("AXCV", (A, X, C, V)):
        assert np.array_equal(f64(t), v[n].astype(np.float64)), f"{n} is not bfloat16-exact"
    print(f"reference vectors {case}", flush=True)
    Y, st = parallel_jagged(A[..., :L].contiguous(), X[..., :L].contiguous(), C[..., :L].contiguous(),
                            V[..., :L].contiguous(), block_len=bl, state_dtype=torch.float32)
    assert_close(f64(Y), v["Y"], BF16_ATOL, BF16_RTOL, "Y")
    assert st.i == i_ref
    assert_close(f64(st.h_loc), v["h_loc"], F32_ATOL, F32_RTOL, "h_loc")
    assert_close(f64(st.r_pref), v["r_pref"], F32_ATOL, F32_RTOL, "r_pref")
    assert_close(f64(st.c_prev_loc), v["c_prev_loc"], F32_ATOL, F32_RTOL, "c_prev_loc")
    for k in range(steps):
        t = L + k
        y, st = step_jagged(A[:, :, t].float(), X[..., t], C[..., t], V[..., t], st, inplace=True)
        assert_close(f64(y), v["y_steps"][..., k], BF16_ATOL, BF16_RTOL, f"decode step {k}")
