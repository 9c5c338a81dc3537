"""``phalanx_mix``: the Phalanx mixing stage as one op on the layer's ``[B, L, features]`` tensors.

    out = btp(sigmoid(a_logits), sigmoid(b_logits) * v) * c + v

Forward is a single HIP kernel that reads each projection output once, in place, and writes the
result once (no transposing copies, no intermediate tensors). It fuses what the reference does in
separate PyTorch ops around its BTP kernel (spear/nn/phalanx/swr.py:166-221, 311-327 and the
``.contiguous()`` calls of spear/ops/btp/interface.py:186-187).

Backward is a second fused kernel (every operand read once, every gradient written once), including
the sum of the ``b`` / ``c`` gradients over the heads that share a kv head, for any
``heads % kv_heads == 0``: groups of 1, 2, 4 or 8 heads are summed inside a wavefront, other group
sizes through LDS (spear/nn/phalanx/swr.py:21-126 accepts every such grouping).
"""

from __future__ import annotations

import torch
import torch.library

from spear_amd import _btp

from .interface import _plain_eager, lib, register_traceable_op

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
        da, db, dc, dv = (torch.empty_like(t) for t in (a_logits, b_logits, c, v))
        torch.ops.spear_btp.mix_backward(a_logits, b_logits, c, v, dout.contiguous(), da, db, dc, dv, H, Hkv)
        return da, db, dc, dv, None, None


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
        heads: number of heads; head_dim is 16.
        kv_heads: number of shared b/c heads (default ``heads``); head ``h`` uses ``h // (heads // kv_heads)``.

    All tensors bf16 or fp16, ``L`` a multiple of 16. Returns ``[B, L, heads*16]`` in the same dtype.
    """
    kv = heads if kv_heads is None else kv_heads
    operands = (a_logits.contiguous(), b_logits.contiguous(), c.contiguous(), v.contiguous())
    return _run_node(_PhalanxMix, operands, heads, kv, False)


def _run_node(python_node, operands, heads: int, kv_heads: int, qkv_gate: bool) -> torch.Tensor:
    """The mixing stage on contiguous operands in the kernel's order. Plain eager tensors that need gradients go
    through the autograd node compiled into the binding (``mix_autograd``: same kernels, same bits, no Python frames
    between autograd and the C ABI); under torch.compile, a dispatch or function mode, a functorch transform or with
    tensor subclasses the Python node over the traceable custom ops runs."""
    if torch.is_grad_enabled() and any(t.requires_grad for t in operands) and _plain_eager(*operands):
        return _btp.load_extension().mix_autograd(*operands, int(heads), int(kv_heads), qkv_gate)
    return python_node.apply(*operands, heads, kv_heads)


class _BtpQkv(torch.autograd.Function):
    """Operands in the kernel's order: gate, k, q, v."""

    @staticmethod
    def forward(ctx, gate, k, q, v, heads: int, kv_heads: int):
        out = torch.empty_like(v)
        torch.ops.spear_btp.qkv_forward(gate, k, q, v, out, heads, kv_heads)
        ctx.save_for_backward(gate, k, q, v)
        ctx.heads, ctx.kv_heads = heads, kv_heads
        return out

    @staticmethod
    def backward(ctx, dout):
        gate, k, q, v = ctx.saved_tensors
        dgate, dk, dq, dv = (torch.empty_like(t) for t in (gate, k, q, v))
        torch.ops.spear_btp.qkv_backward(gate, k, q, v, dout.contiguous(), dgate, dk, dq, dv, ctx.heads, ctx.kv_heads)
        return dgate, dk, dq, dv, None, None


def btp_qkv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """The operator in linear-attention terms, time-major:

        out = q * btp(exp(gate), k * v) + v

    one fused kernel forward and one backward (``dq, dk, dv, dgate``), no transposes.

    Args:
        q, k: ``[B, L, kv_heads, 16]`` bf16 / fp16 (``kv_heads`` divides ``heads``; head ``h`` uses q/k of kv head
            ``h // (heads // kv_heads)``).
        v: ``[B, L, heads, 16]``, same dtype; ``L`` a multiple of 16.
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
    if Hkv == 0 or H % Hkv != 0:
        raise RuntimeError("heads must be divisible by kv_heads.")
    operands = (gate.contiguous(), k.reshape(B, L, Hkv * 16).contiguous(), q.reshape(B, L, Hkv * 16).contiguous(),
                v.reshape(B, L, H * 16).contiguous())
    return _run_node(_BtpQkv, operands, H, Hkv, True).view(B, L, H, 16)
