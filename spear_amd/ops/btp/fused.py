"""``phalanx_mix``: the Phalanx mixing stage as one op on the layer's ``[B, L, features]`` tensors.

    out = btp(sigmoid(a_logits), sigmoid(b_logits) * v) * c + v

Forward is a single HIP kernel that reads each projection output once, in place, and writes the
result once (no transposing copies, no intermediate tensors). It fuses what the reference does in
separate PyTorch ops around its BTP kernel (spear/nn/phalanx/swr.py:166-221, 311-327 and the
``.contiguous()`` calls of spear/ops/btp/interface.py:186-187).

Backward is a second fused kernel (reverse walk through time, every operand read once, every
gradient written once), including the sum of the ``b`` / ``c`` gradients over the heads that share
a kv head when a group has 2, 4 or 8 heads. Larger groups span several wavefronts; that case
recomputes the gates with PyTorch ops in the ``[B, H, 16, L]`` layout and calls the stand-alone
BTP kernels.
"""

from __future__ import annotations

import torch
import torch.library

from spear_amd import _btp

from .interface import lib, register_traceable_op

__all__ = ["phalanx_mix", "btp_qkv"]


def _mix_forward_impl(
    a_logits: torch.Tensor, b_logits: torch.Tensor, c: torch.Tensor, v: torch.Tensor, out: torch.Tensor,
    heads: int, kv_heads: int,
) -> None:
    _btp.load_extension().mix_forward(a_logits, b_logits, c, v, out, heads, kv_heads)


def _mix_forward_fake(
    a_logits: torch.Tensor, b_logits: torch.Tensor, c: torch.Tensor, v: torch.Tensor, out: torch.Tensor,
    heads: int, kv_heads: int,
) -> None:
    return None


def _mix_backward_impl(
    a_logits: torch.Tensor, b_logits: torch.Tensor, c: torch.Tensor, v: torch.Tensor, dout: torch.Tensor,
    da: torch.Tensor, db: torch.Tensor, dc: torch.Tensor, dv: torch.Tensor, heads: int, kv_heads: int,
) -> None:
    _btp.load_extension().mix_backward(a_logits, b_logits, c, v, dout, da, db, dc, dv, heads, kv_heads)


def _mix_backward_fake(
    a_logits: torch.Tensor, b_logits: torch.Tensor, c: torch.Tensor, v: torch.Tensor, dout: torch.Tensor,
    da: torch.Tensor, db: torch.Tensor, dc: torch.Tensor, dv: torch.Tensor, heads: int, kv_heads: int,
) -> None:
    return None


register_traceable_op(lib, "mix_forward", _mix_forward_impl, _mix_forward_fake, mutates_args=["out"])
register_traceable_op(
    lib, "mix_backward", _mix_backward_impl, _mix_backward_fake, mutates_args=["da", "db", "dc", "dv"]
)


def _qkv_forward_impl(
    gate: torch.Tensor, k: torch.Tensor, q: torch.Tensor, v: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int
) -> None:
    _btp.load_extension().mix_forward(gate, k, q, v, out, heads, kv_heads, True)


def _qkv_forward_fake(
    gate: torch.Tensor, k: torch.Tensor, q: torch.Tensor, v: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int
) -> None:
    return None


def _qkv_backward_impl(
    gate: torch.Tensor, k: torch.Tensor, q: torch.Tensor, v: torch.Tensor, dout: torch.Tensor,
    dgate: torch.Tensor, dk: torch.Tensor, dq: torch.Tensor, dv: torch.Tensor, heads: int, kv_heads: int,
) -> None:
    _btp.load_extension().mix_backward(gate, k, q, v, dout, dgate, dk, dq, dv, heads, kv_heads, [], True)


def _qkv_backward_fake(
    gate: torch.Tensor, k: torch.Tensor, q: torch.Tensor, v: torch.Tensor, dout: torch.Tensor,
    dgate: torch.Tensor, dk: torch.Tensor, dq: torch.Tensor, dv: torch.Tensor, heads: int, kv_heads: int,
) -> None:
    return None


register_traceable_op(lib, "qkv_forward", _qkv_forward_impl, _qkv_forward_fake, mutates_args=["out"])
register_traceable_op(
    lib, "qkv_backward", _qkv_backward_impl, _qkv_backward_fake, mutates_args=["dgate", "dk", "dq", "dv"]
)


def _to_heads(t: torch.Tensor, heads: int) -> torch.Tensor:
    """[B, L, heads*16] -> [B, heads, 16, L] (a view)."""
    B, L, _ = t.shape
    return t.view(B, L, heads, 16).permute(0, 2, 3, 1)


def _from_heads(t: torch.Tensor) -> torch.Tensor:
    """[B, heads, 16, L] -> [B, L, heads*16] (materialised)."""
    B, H, D, L = t.shape
    return t.permute(0, 3, 1, 2).reshape(B, L, H * D)


class _PhalanxMix(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a_logits, b_logits, c, v, heads: int, kv_heads: int):
        out = torch.empty_like(v)
        torch.ops.spear_btp.mix_forward(a_logits, b_logits, c, v, out, heads, kv_heads)
        ctx.save_for_backward(a_logits, b_logits, c, v)
        ctx.heads, ctx.kv_heads = heads, kv_heads
        return out

    @staticmethod
    def backward(ctx, dout):
        a_logits, b_logits, c, v = ctx.saved_tensors
        H, Hkv = ctx.heads, ctx.kv_heads
        groups = H // Hkv
        dout = dout.contiguous()
        if groups in (1, 2, 4, 8) and (groups < 8 or H % 8 == 0):
            da, db, dc, dv = (torch.empty_like(t) for t in (a_logits, b_logits, c, v))
            torch.ops.spear_btp.mix_backward(a_logits, b_logits, c, v, dout, da, db, dc, dv, H, Hkv)
            return da, db, dc, dv, None, None

        # Head groups that span wavefronts: gates recomputed with PyTorch ops, stand-alone kernels for the
        # recurrence. The decay and the gated input are rounded to the tensors' 16-bit type on the way (the
        # stand-alone op takes 16-bit operands), so these gradients differ from the fused kernel's in the last
        # bits of that rounding.

        B, L, _ = v.shape
        dt = v.dtype

        def expand(t):  # [B, Hkv, 16, L] -> [B, H, 16, L]
            return t.repeat_interleave(groups, dim=1) if groups > 1 else t

        A32 = torch.sigmoid(a_logits.float()).transpose(1, 2)            # [B, H, L]
        G32 = expand(torch.sigmoid(_to_heads(b_logits, Hkv).float()))    # [B, H, 16, L]
        C32 = expand(_to_heads(c, Hkv).float())
        V32 = _to_heads(v, H).float()
        dO = _to_heads(dout, H).float()

        A = A32.to(dt).contiguous()
        X = (G32 * V32).to(dt).contiguous()
        ck = torch.empty((B, H, L // 16, 16), device=v.device, dtype=torch.float32)
        h = torch.empty((B, H, 16, L), device=v.device, dtype=torch.float32)
        torch.ops.spear_btp.forward(A, X, h, ck, 2, 32)
        dh = (dO * C32).contiguous()
        dX = torch.empty_like(X)
        dA = torch.empty((B, H, L), device=v.device, dtype=torch.float32)
        torch.ops.spear_btp.backward(A, X, dh, ck, dX, dA, 2, 32)
        dX32 = dX.float()

        dC = dO * h
        dV = dO + dX32 * G32
        dB = dX32 * V32 * G32 * (1.0 - G32)
        da = (dA * A32 * (1.0 - A32)).transpose(1, 2)
        if groups > 1:
            dC = dC.view(B, Hkv, groups, 16, L).sum(2)
            dB = dB.view(B, Hkv, groups, 16, L).sum(2)
        return (
            da.to(dt).contiguous(),
            _from_heads(dB).to(dt),
            _from_heads(dC).to(dt),
            _from_heads(dV).to(dt),
            None,
            None,
        )


def phalanx_mix(
    a_logits: torch.Tensor,
    b_logits: torch.Tensor,
    c: torch.Tensor,
    v: torch.Tensor,
    heads: int,
    kv_heads: int | None = None,
) -> torch.Tensor:
    """Fused mixing stage of the Phalanx layer.

    Args:
        a_logits: ``[B, L, heads]`` decay logits (``proj_a`` output).
        b_logits: ``[B, L, kv_heads*16]`` input-gate logits (``proj_b`` output).
        c: ``[B, L, kv_heads*16]`` output gate (``proj_c`` output).
        v: ``[B, L, heads*16]`` values (``proj_v`` output).
        heads: number of heads (a multiple of 4); head_dim is 16.
        kv_heads: number of shared b/c heads (default ``heads``); head ``h`` uses ``h // (heads // kv_heads)``.

    All tensors bf16 or fp16, ``L`` a multiple of 16. Returns ``[B, L, heads*16]`` in the same dtype.
    """
    kv = heads if kv_heads is None else kv_heads
    return _PhalanxMix.apply(a_logits.contiguous(), b_logits.contiguous(), c.contiguous(), v.contiguous(), heads, kv)


class _BtpQkv(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, gate, heads: int, kv_heads: int):
        out = torch.empty_like(v)
        torch.ops.spear_btp.qkv_forward(gate, k, q, v, out, heads, kv_heads)
        ctx.save_for_backward(q, k, v, gate)
        ctx.heads, ctx.kv_heads = heads, kv_heads
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, gate = ctx.saved_tensors
        dq, dk, dv, dgate = (torch.empty_like(t) for t in (q, k, v, gate))
        torch.ops.spear_btp.qkv_backward(gate, k, q, v, dout.contiguous(), dgate, dk, dq, dv, ctx.heads, ctx.kv_heads)
        return dq, dk, dv, dgate, None, None


def btp_qkv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """The operator in linear-attention terms, time-major:

        out = q * btp(exp(gate), k * v) + v

    one fused kernel forward and one backward (``dq, dk, dv, dgate``), no transposes.

    Args:
        q, k: ``[B, L, kv_heads, 16]`` bf16 / fp16 (``kv_heads`` divides ``heads``; ``heads // kv_heads`` in
            1, 2, 4, 8; head ``h`` uses q/k of kv head ``h // (heads // kv_heads)``).
        v: ``[B, L, heads, 16]``, same dtype; ``heads`` a multiple of 4, ``L`` a multiple of 16.
        gate: ``[B, L, heads]`` float32 log-decay (``<= 0``, e.g. ``-softplus(logit)``); the decay
            ``exp(gate)`` is formed in fp32 inside the kernel, and the gradient is w.r.t. ``gate``.

    Returns ``[B, L, heads, 16]`` in ``v``'s dtype. This is what the Phalanx layer computes
    (spear/nn/phalanx/swr.py:196-221, 311-327) with ``k = sigmoid(proj_b(x))``, ``q = proj_c(x)``,
    ``gate = log sigmoid(proj_a(x))``.
    """
    if v.dim() != 4 or v.shape[-1] != 16 or q.dim() != 4 or q.shape != k.shape or q.shape[-1] != 16:
        raise RuntimeError("q, k must be [B, L, kv_heads, 16] and v [B, L, heads, 16].")
    B, L, H, _ = v.shape
    Hkv = q.shape[2]
    if Hkv == 0 or H % Hkv != 0 or H // Hkv not in (1, 2, 4, 8) or (H // Hkv == 8 and H % 8 != 0):
        raise RuntimeError("heads / kv_heads must be 1, 2, 4 or 8.")
    out = _BtpQkv.apply(
        q.reshape(B, L, Hkv * 16).contiguous(), k.reshape(B, L, Hkv * 16).contiguous(),
        v.reshape(B, L, H * 16).contiguous(), gate.contiguous(), H, Hkv,
    )
    return out.view(B, L, H, 16)
