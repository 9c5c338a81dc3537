"""The layer-layout decode step (spear_phalanx_mix_step, phalanx_step / phalanx_prefill): one token of the
Phalanx mixing stage on the projections' [B, features] outputs with the fp32 streaming state, against the
float64 oracle (oracle.jagged_oracle.layer_step), against the layer's own forward, and as a HIP graph that is
replayed once per token."""

import numpy as np
import pytest
import torch

from helpers import BF16_ATOL, BF16_RTOL, F32_ATOL, F32_RTOL, assert_close, f64
from oracle import jagged_oracle as jag

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def token_inputs(B, H, Hkv, n, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(B, H, generator=g).to(dtype), torch.randn(B, Hkv * 16, generator=g).to(dtype),
             torch.randn(B, Hkv * 16, generator=g).to(dtype), torch.randn(B, H * 16, generator=g).to(dtype)) for _ in range(n)]


@pytest.mark.parametrize("B,H,Hkv,n", [(1, 4, 4, 35), (3, 8, 2, 20), (2, 32, 32, 18), (5, 12, 3, 33), (2, 64, 8, 17)])
@pytest.mark.parametrize("device_positions", [True, False], ids=["pos_on_device", "host_boundary"])
def test_step_kernel_matches_oracle_over_block_boundaries(B, H, Hkv, n, device_positions):
    from spear_amd import _btp

    toks = token_inputs(B, H, Hkv, n, seed=9000 + H + n)
    h = torch.zeros(B, H, 16, device=DEV)
    r = torch.ones(B, H, device=DEV)
    cp = torch.zeros(B, H, 16, device=DEV)
    pos = torch.zeros(B, device=DEV, dtype=torch.int32) if device_positions else None
    ref = jag.zero_state(B, H, 16, 16)
    print(f"layer step B={B} H={H} Hkv={Hkv} n={n} device_positions={device_positions}", flush=True)
    for t, (a, b, c, v) in enumerate(toks):
        out = torch.full((B, H * 16), float("nan"), device=DEV, dtype=torch.bfloat16)
        _btp.mix_step(a.to(DEV), b.to(DEV), c.to(DEV), v.to(DEV), out, h, r, cp, pos, (t + 1) % 16 == 0, 16, H, Hkv)
        want, ref = jag.layer_step(f64(a), f64(b), f64(c), f64(v), ref, H, Hkv)
        assert_close(f64(out), want, BF16_ATOL, BF16_RTOL, f"out[{t}]")
        # the state is fp32 and never rounded to 16 bits: it follows the oracle at the fp32 bound
        assert_close(f64(h), ref.h_loc, F32_ATOL, F32_RTOL, f"h[{t}]")
        assert_close(f64(r), ref.r_pref, F32_ATOL, F32_RTOL, f"r[{t}]")
        assert_close(f64(cp), ref.c_prev_loc, F32_ATOL, F32_RTOL, f"c_prev[{t}]")
        if pos is not None:
            assert pos.tolist() == [(t + 1) % 16] * B


def test_batch_rows_at_different_block_positions():
    """With positions on the device every batch row closes its block when its own position says so."""
    from spear_amd import _btp

    B, H = 4, 8
    offsets = [0, 5, 15, 9]
    toks = token_inputs(B, H, H, 20, seed=9100)
    h = torch.zeros(B, H, 16, device=DEV)
    r = torch.ones(B, H, device=DEV)
    cp = torch.zeros(B, H, 16, device=DEV)
    pos = torch.tensor(offsets, device=DEV, dtype=torch.int32)
    refs = [jag.zero_state(1, H, 16, 16) for _ in range(B)]
    for b_, off in enumerate(offsets):
        refs[b_].i = off
    for t, (a, b, c, v) in enumerate(toks):
        out = torch.empty(B, H * 16, device=DEV, dtype=torch.bfloat16)
        _btp.mix_step(a.to(DEV), b.to(DEV), c.to(DEV), v.to(DEV), out, h, r, cp, pos, False, 16, H, H)
        for b_ in range(B):
            want, refs[b_] = jag.layer_step(f64(a[b_:b_ + 1]), f64(b[b_:b_ + 1]), f64(c[b_:b_ + 1]), f64(v[b_:b_ + 1]), refs[b_], H, H)
            assert_close(f64(out[b_:b_ + 1]), want, BF16_ATOL, BF16_RTOL, f"out[{t}][{b_}]")
    assert pos.tolist() == [(o + 20) % 16 for o in offsets]


def _layer(dim=128, kv_heads=None, seed=3):
    from spear_amd import Phalanx

    torch.manual_seed(seed)
    return Phalanx(dim=dim, length=64, method="fused", dtype=torch.bfloat16, kv_heads=kv_heads).to(DEV)


# (dim 64, B 1) and (dim 192, B 3): the rows a[t] of the tail's [tokens, B, H] logits start on 8- and 2-byte
# boundaries there (B * H * 2 bytes per token is not a multiple of 16)
@pytest.mark.parametrize("L,kv_heads,dim,B", [(48, None, 128, 3), (37, 2, 128, 3), (16, None, 128, 3), (5, None, 128, 3),
                                              (37, None, 64, 1), (37, None, 192, 3), (29, 6, 192, 1)])
def test_stepping_a_layer_equals_its_forward_and_prefill_hands_over(L, kv_heads, dim, B):
    """Token t of phalanx_step equals position t of the layer's forward on the whole sequence (both run the same
    projections; the mixing stage is the fused kernel there and the step kernel here), and prefill(first part) +
    steps continues exactly like stepping from the start."""
    from spear_amd.nn.phalanx.inference import PhalanxStepState, phalanx_prefill, phalanx_step

    layer = _layer(dim=dim, kv_heads=kv_heads)
    n_more = 21
    x = torch.randn(B, L + n_more, dim, generator=torch.Generator().manual_seed(L)).bfloat16().to(DEV)
    Lw = ((L + n_more) // 16) * 16
    with torch.no_grad():
        whole = layer(x[:, :Lw]).float()                     # forward needs whole blocks
    state = PhalanxStepState.zeros(B, layer.heads, DEV)
    stepped = torch.stack([phalanx_step(layer, x[:, t], state) for t in range(L + n_more)], dim=1).float()
    # two bf16 roundings apart at most (the mixing stage's output, then proj_out): the bf16 bound on the output scale
    scale = float(whole.abs().max())
    assert float((stepped[:, :Lw] - whole).abs().max()) <= 2e-2 * scale

    y, st = phalanx_prefill(layer, x[:, :L])
    assert y.shape == (B, L, dim)
    assert float((y.float() - stepped[:, :L]).abs().max()) <= 2e-2 * scale
    # the prefill projects the prompt as one matrix product and stepping projects token by token: the library may
    # sum those in another order, so the two states agree to the 16-bit rounding of the projections, not bit for bit
    ref_state = PhalanxStepState.zeros(B, layer.heads, DEV)
    for t in range(L):
        phalanx_step(layer, x[:, t], ref_state)
    assert st.pos.tolist() == ref_state.pos.tolist() == [L % 16] * B
    for name in ("h_loc", "r_pref", "c_prev_loc"):
        got, want = getattr(st, name), getattr(ref_state, name)
        assert float((got - want).abs().max()) <= 2e-2 * max(1.0, float(want.abs().max())), name
    cont = torch.stack([phalanx_step(layer, x[:, t], st) for t in range(L, L + n_more)], dim=1).float()
    assert float((cont - stepped[:, L:]).abs().max()) <= 2e-2 * scale


@pytest.mark.parametrize("B,H,Hkv,L", [(2, 4, 4, 16), (3, 8, 2, 48), (1, 32, 32, 128), (2, 12, 3, 272), (1, 64, 8, 2048),
                                       (2, 6, 2, 80), (1, 3, 1, 48), (2, 16, 1, 64)])
def test_prefill_kernel_leaves_the_state_that_stepping_reaches(B, H, Hkv, L):
    """spear_phalanx_mix_prefill on [B, L, features] against L calls of the step kernel on the same tensors: the
    hand-over state is the same fp32 arithmetic in the same order, so it is equal bit for bit; the outputs agree
    with the float64 oracle, and the forward entry point (no state) gives the same output."""
    from spear_amd import _btp

    g = torch.Generator().manual_seed(9200 + L + H)
    a = torch.randn(B, L, H, generator=g).bfloat16().to(DEV)
    b = torch.randn(B, L, Hkv * 16, generator=g).bfloat16().to(DEV)
    c = torch.randn(B, L, Hkv * 16, generator=g).bfloat16().to(DEV)
    v = torch.randn(B, L, H * 16, generator=g).bfloat16().to(DEV)
    out, plain = torch.empty_like(v), torch.empty_like(v)
    tail = torch.full((B, H, 16), float("nan"), device=DEV)
    print(f"mix prefill B={B} H={H} Hkv={Hkv} L={L}", flush=True)
    _btp.mix_forward(a, b, c, v, out, H, Hkv, c_prev_tail=tail)
    _btp.mix_forward(a, b, c, v, plain, H, Hkv)
    assert torch.equal(out, plain)

    h = torch.zeros(B, H, 16, device=DEV)
    r = torch.ones(B, H, device=DEV)
    cp = torch.zeros(B, H, 16, device=DEV)
    pos = torch.zeros(B, device=DEV, dtype=torch.int32)
    stepped = torch.empty_like(v)
    # stepped[:, t] is a strided view: step into a dense row and copy
    row = torch.empty(B, H * 16, device=DEV, dtype=torch.bfloat16)
    for t in range(L):
        _btp.mix_step(a[:, t].contiguous(), b[:, t].contiguous(), c[:, t].contiguous(), v[:, t].contiguous(), row,
                      h, r, cp, pos, False, 16, H, Hkv)
        stepped[:, t] = row
    assert torch.equal(tail, cp), "hand-over state"
    assert float(h.abs().max()) == 0.0 and torch.equal(r, torch.ones_like(r)) and pos.tolist() == [0] * B
    assert_close(f64(out), f64(stepped), BF16_ATOL, BF16_RTOL, "prefill output vs stepping")
    if L <= 272:
        ref = jag.zero_state(B, H, 16, 16)
        for t in range(L):
            want, ref = jag.layer_step(f64(a[:, t]), f64(b[:, t]), f64(c[:, t]), f64(v[:, t]), ref, H, Hkv)
            assert_close(f64(out[:, t]), want, BF16_ATOL, BF16_RTOL, f"out[{t}]")
        assert_close(f64(tail), ref.c_prev_loc, F32_ATOL, F32_RTOL, "c_prev_tail")


def test_prefill_entry_point_refuses_the_qkv_form_and_a_wrong_state():
    from spear_amd import _btp

    B, H, L = 1, 4, 16
    a = torch.zeros(B, L, H, device=DEV, dtype=torch.bfloat16)
    kv = torch.zeros(B, L, H * 16, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="float32"):
        _btp.mix_forward(a, kv, kv, kv, torch.empty_like(kv), H, H, c_prev_tail=torch.zeros(B, H, 16, device=DEV).bfloat16())
    with pytest.raises(RuntimeError, match="layer form"):
        _btp.mix_forward(a.float(), kv, kv, kv, torch.empty_like(kv), H, H, qkv_gate=True, c_prev_tail=torch.zeros(B, H, 16, device=DEV))


def test_one_graph_replayed_per_token_reproduces_eager_decoding():
    """The whole layer step (projections, step kernel, position update, output projection) recorded once and
    replayed for every token, across block boundaries, with eager work between the replays."""
    from spear_amd.nn.phalanx.inference import PhalanxStepState, phalanx_step

    layer = _layer(dim=256, seed=5)
    B, n = 4, 40
    xs = torch.randn(n, B, 256, generator=torch.Generator().manual_seed(77)).bfloat16().to(DEV)
    eager_state = PhalanxStepState.zeros(B, layer.heads, DEV)
    eager = [phalanx_step(layer, xs[t], eager_state).clone() for t in range(n)]

    state = PhalanxStepState.zeros(B, layer.heads, DEV)
    x_buf = torch.zeros(B, 256, device=DEV, dtype=torch.bfloat16)
    y_buf = torch.zeros(B, 256, device=DEV, dtype=torch.bfloat16)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                             # warm-up on the capture stream, on scratch state
        phalanx_step(layer, x_buf, PhalanxStepState.zeros(B, layer.heads, DEV), out=y_buf)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        phalanx_step(layer, x_buf, state, out=y_buf)
    # the capture itself does not run the step: the state is still the zero state
    assert float(state.h_loc.abs().max()) == 0.0 and state.pos.tolist() == [0] * B
    for t in range(n):
        x_buf.copy_(xs[t])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_buf, eager[t]), f"replay {t}"
        _ = (xs[t].float() @ xs[t].float().T).sum().item()    # unrelated eager work between replays
    assert state.pos.tolist() == [n % 16] * B
    assert torch.equal(state.h_loc, eager_state.h_loc) and torch.equal(state.c_prev_loc, eager_state.c_prev_loc)


def test_step_rejects_bad_arguments():
    from spear_amd import _btp

    B, H = 2, 4
    a, b, c, v = (t.to(DEV) for t in token_inputs(B, H, H, 1, seed=1)[0])
    out = torch.empty_like(v)
    h, r, cp = torch.zeros(B, H, 16, device=DEV), torch.ones(B, H, device=DEV), torch.zeros(B, H, 16, device=DEV)
    with pytest.raises(RuntimeError, match="state must be float32"):
        _btp.mix_step(a, b, c, v, out, h.bfloat16(), r, cp, None, False, 16, H, H)
    with pytest.raises(RuntimeError, match="pos must be int32"):
        _btp.mix_step(a, b, c, v, out, h, r, cp, torch.zeros(B, device=DEV), False, 16, H, H)
    with pytest.raises(RuntimeError, match="shape"):
        _btp.mix_step(a, b, c, v, out, h, r[:1], cp, None, False, 16, H, H)
    with pytest.raises(RuntimeError, match="block_len must be positive"):
        _btp.mix_step(a, b, c, v, out, h, r, cp, None, False, 0, H, H)
