"""The layer's linear projections with a backward pass shaped for long token axes.

The Phalanx layer (spear/nn/phalanx/swr.py:166-175, 271) is five ``nn.Linear`` calls around the
mixing stage. With ``M = B*L`` tokens their weight gradients are ``[N, M] x [M, K]`` products whose
output is a few hundred columns wide while the reduction runs over 10^5 tokens: as one GEMM that is a
few dozen output tiles for 256 compute units. Here the token axis is cut into ``S`` slices that are
multiplied as one batched GEMM with fp32 partial results and then summed (the same fp32 accumulation,
associated differently). The four input projections also share one backward: their input gradients
accumulate in one buffer through the GEMM's own ``beta = 1`` epilogue instead of four products and
three additions. ``project_and_mix`` goes further for the fused mixing stage: its backward kernel writes the
four gradients side by side into one ``[B, L, ld]`` buffer, which is the gradient of the concatenated
projection, so input and weight gradients are one GEMM each against the stacked weights (the forward stays
four GEMMs, which measured faster than one wide one); and the kernel leaves the column sums of the gate
gradients (the three bias gradients) per tile of 64 time steps, so they are not read again to be summed.

Short token axes gain nothing (their step is bound by launch overhead, of which this path has more), so
the layer uses these functions from 8192 tokens on (``pays_off``).

Forward results are those of ``torch.nn.functional.linear``. Parameters stay in the layer's
``nn.Linear`` modules; these functions only take their tensors.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

__all__ = ["weight_grad", "input_projections", "linear", "pays_off", "project_and_mix", "packed_columns"]

_TILE = 128           # output tile edge the slice count is sized against
_TARGET_TILES = 1024  # about four tiles per compute unit
_MIN_SLICE_ROWS = 1024
_MAX_SLICES = 64
_MIN_TOKENS = 8192    # below this a step is bound by launches, and these functions add a few


def pays_off(x: torch.Tensor) -> bool:
    """Whether ``x[..., K]`` has enough tokens for the sliced backward to beat plain ``nn.Linear``."""
    return x.is_cuda and x.numel() // x.shape[-1] >= _MIN_TOKENS


def slice_count(M: int, N: int, K: int) -> int:
    """How many slices the token axis of an ``[N, M] x [M, K]`` product is cut into."""
    tiles = -(-N // _TILE) * -(-K // _TILE)
    s = 1
    while s < _MAX_SLICES and tiles * s < _TARGET_TILES and M % (2 * s) == 0 and M // (2 * s) >= _MIN_SLICE_ROWS:
        s *= 2
    return s


@torch.library.custom_op("spear_amd::weight_grad", mutates_args=())
def weight_grad(dy: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """``dy[M, N]^T @ x[M, K] -> [N, K]`` in ``dy``'s dtype, accumulated in fp32."""
    M, N = dy.shape
    K = x.shape[1]
    s = slice_count(M, N, K) if dy.is_cuda and dy.dtype in (torch.bfloat16, torch.float16) else 1
    if s == 1:
        return dy.t() @ x
    dy3 = dy.contiguous().view(s, M // s, N)
    x3 = x.contiguous().view(s, M // s, K)
    return torch.bmm(dy3.transpose(1, 2), x3, out_dtype=torch.float32).sum(0).to(dy.dtype)


@weight_grad.register_fake
def _(dy, x):
    return dy.new_empty((dy.shape[1], x.shape[1]))


class _InputProjections(torch.autograd.Function):
    """x[M, K] -> (x W_a^T + b_a, x W_b^T + b_b, x W_c^T + b_c, x W_v^T)."""

    @staticmethod
    def forward(ctx, x, w_a, b_a, w_b, b_b, w_c, b_c, w_v):
        ctx.save_for_backward(x, w_a, w_b, w_c, w_v)
        return F.linear(x, w_a, b_a), F.linear(x, w_b, b_b), F.linear(x, w_c, b_c), F.linear(x, w_v)

    @staticmethod
    def backward(ctx, d_a, d_b, d_c, d_v):
        x, w_a, w_b, w_c, w_v = ctx.saved_tensors
        need = ctx.needs_input_grad
        pairs = [(d, w) for d, w in ((d_v, w_v), (d_b, w_b), (d_c, w_c), (d_a, w_a)) if d is not None]
        dx = None
        if need[0] and pairs:
            dx = pairs[0][0] @ pairs[0][1]
            for d, w in pairs[1:]:
                dx.addmm_(d, w)

        def wgrad(d, wanted):
            return weight_grad(d, x) if wanted and d is not None else None

        def bgrad(d, wanted):
            return d.sum(0) if wanted and d is not None else None

        return (dx, wgrad(d_a, need[1]), bgrad(d_a, need[2]), wgrad(d_b, need[3]), bgrad(d_b, need[4]),
                wgrad(d_c, need[5]), bgrad(d_c, need[6]), wgrad(d_v, need[7]))


class _Linear(torch.autograd.Function):
    """x[M, K] -> x W^T (no bias)."""

    @staticmethod
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return F.linear(x, w)

    @staticmethod
    def backward(ctx, d):
        x, w = ctx.saved_tensors
        return (d @ w if ctx.needs_input_grad[0] else None, weight_grad(d, x) if ctx.needs_input_grad[1] else None)


def packed_columns(heads: int, kv_heads: int) -> tuple[dict[str, tuple[int, int]], int]:
    """Column blocks ``name -> (first column, width)`` of the four projections' outputs laid side by side
    as ``[b | c | v | a | padding]``, and the padded row length (a multiple of 64 elements, so that every
    row of the packed buffer starts on a 128-byte line)."""
    Fkv, F = kv_heads * 16, heads * 16
    cols = {"b": (0, Fkv), "c": (Fkv, Fkv), "v": (2 * Fkv, F), "a": (2 * Fkv + F, heads)}
    used = 2 * Fkv + F + heads
    return cols, -(-used // 64) * 64


@torch.library.custom_op("spear_amd::mix_backward_packed", mutates_args=())
def _mix_backward_packed(
    a_logits: torch.Tensor, b_logits: torch.Tensor, c: torch.Tensor, v: torch.Tensor, dout: torch.Tensor,
    heads: int, kv_heads: int,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Backward of the fused mixing stage with its four gradients written side by side into one
    ``[B, L, ld]`` buffer (``packed_columns``; padding columns zero), and the sums over all tokens of the
    ``a``, ``b`` and ``c`` blocks: ``(packed, da.sum, db.sum, dc.sum)``."""
    from spear_amd import _btp

    B, L, _ = v.shape
    cols, ld = packed_columns(heads, kv_heads)
    packed = torch.empty((B, L, ld), device=v.device, dtype=v.dtype)
    used = cols["a"][0] + cols["a"][1]
    if used < ld:
        packed[..., used:].zero_()
    da, db, dc, dv = (packed[..., cols[k][0]:cols[k][0] + cols[k][1]] for k in "abcv")
    rows = _btp.mix_backward_sum_rows(B, L, heads)
    sums = [torch.empty((rows, t.shape[-1]), device=v.device, dtype=torch.float32) for t in (a_logits, b_logits, c)]
    _btp.mix_backward(a_logits, b_logits, c, v, dout, da, db, dc, dv, heads, kv_heads, sums=tuple(sums))
    return (packed, *(s.sum(0).to(v.dtype) for s in sums))


@_mix_backward_packed.register_fake
def _(a_logits, b_logits, c, v, dout, heads, kv_heads):
    B, L, _ = v.shape
    packed = v.new_empty((B, L, packed_columns(heads, kv_heads)[1]))
    return (packed, *(t.new_empty((t.shape[-1],)) for t in (a_logits, b_logits, c)))


class _ProjectAndMix(torch.autograd.Function):
    """x[B, L, K] -> mixing stage of its four projections, [B, L, heads*16]."""

    @staticmethod
    def forward(ctx, x, w_a, b_a, w_b, b_b, w_c, b_c, w_v, heads: int, kv_heads: int):
        a, b, c, v = F.linear(x, w_a, b_a), F.linear(x, w_b, b_b), F.linear(x, w_c, b_c), F.linear(x, w_v)
        out = torch.empty_like(v)
        torch.ops.spear_btp.mix_forward(a, b, c, v, out, heads, kv_heads)
        ctx.save_for_backward(x, w_a, w_b, w_c, w_v, a, b, c, v)
        ctx.heads, ctx.kv_heads = heads, kv_heads
        return out

    @staticmethod
    def backward(ctx, dout):
        x, w_a, w_b, w_c, w_v, a, b, c, v = ctx.saved_tensors
        need = ctx.needs_input_grad
        packed, s_a, s_b, s_c = _mix_backward_packed(a, b, c, v, dout.contiguous(), ctx.heads, ctx.kv_heads)
        cols, ld = packed_columns(ctx.heads, ctx.kv_heads)
        x2, d2 = x.reshape(-1, x.shape[-1]), packed.view(-1, ld)
        # one GEMM each against the weights stacked in the buffer's column order
        dx = None
        if need[0]:
            stacked = [w_b, w_c, w_v, w_a]
            pad = ld - (cols["a"][0] + cols["a"][1])
            if pad:
                stacked.append(w_a.new_zeros((pad, w_a.shape[1])))
            dx = (d2 @ torch.cat(stacked)).view(x.shape)
        dw = weight_grad(d2, x2) if any(need[i] for i in (1, 3, 5, 7)) else None

        def rows_of(name, wanted):
            return dw[cols[name][0]:cols[name][0] + cols[name][1]] if wanted else None

        return (dx, rows_of("a", need[1]), s_a if need[2] else None, rows_of("b", need[3]), s_b if need[4] else None,
                rows_of("c", need[5]), s_c if need[6] else None, rows_of("v", need[7]), None, None)


def project_and_mix(x: torch.Tensor, proj_a, proj_b, proj_c, proj_v, heads: int, kv_heads: int) -> torch.Tensor:
    """``phalanx_mix(proj_a(x), proj_b(x), proj_c(x), proj_v(x), heads, kv_heads)`` for ``x[B, L, K]`` with the
    projections' backward of this module and the bias gradients taken from the mixing kernel."""
    import spear_amd.ops.btp.fused  # noqa: F401  (registers torch.ops.spear_btp.mix_forward)

    return _ProjectAndMix.apply(x.contiguous(), proj_a.weight, proj_a.bias, proj_b.weight, proj_b.bias,
                                proj_c.weight, proj_c.bias, proj_v.weight, heads, kv_heads)


def input_projections(x: torch.Tensor, proj_a, proj_b, proj_c, proj_v):
    """The four input projections of ``x[..., K]`` (``nn.Linear`` modules; ``proj_v`` without bias)."""
    lead = x.shape[:-1]
    outs = _InputProjections.apply(
        x.reshape(-1, x.shape[-1]), proj_a.weight, proj_a.bias, proj_b.weight, proj_b.bias,
        proj_c.weight, proj_c.bias, proj_v.weight,
    )
    return tuple(o.view(*lead, o.shape[-1]) for o in outs)


def linear(x: torch.Tensor, proj) -> torch.Tensor:
    """``proj(x)`` for a bias-free ``nn.Linear``."""
    lead = x.shape[:-1]
    out = _Linear.apply(x.reshape(-1, x.shape[-1]), proj.weight)
    return out.view(*lead, out.shape[-1])
