"""``btp(coeff, x, k=2, wpb=None, output_dtype=None)``: the Block Two-Pass operator on MI355X.

Drop-in for the reference's ``spear.ops.btp.interface`` (spear/ops/btp/interface.py): same public
function, same constants, the same two custom ops ``torch.ops.spear_btp.forward`` /
``torch.ops.spear_btp.backward`` (schemas at interface.py:55-120, registered so that
``torch.compile`` can trace through them), and the same autograd contract
(interface.py:126-161): backward returns ``(dA fp32 [B,H,L], dx [B,H,16,L] in x.dtype)``.

Differences that do not change results:
  * the compiled binding (``spear_amd._btp_ext``, the counterpart of ``spear._btp``) is imported on
    first use, so importing this module works before anything is built (the reference imports its
    extension unconditionally, interface.py:16); a call without it raises, there is no fallback;
  * a plain eager call (ordinary tensors, no trace, mode or transform in force) runs the same autograd node
    compiled into the binding (``btp_autograd``) instead of ``_BTPFunction``: same kernels, same results,
    less host time per call;
  * ``dA`` is allocated uninitialised, because the kernel writes every element
    (the reference zero-fills it, interface.py:158);
  * the carry checkpoint is not stored by default, because this backward recomputes the carries:
    the op then receives a zero-element placeholder (its schema requires a tensor) and nothing of
    that size is kept alive for backward. Set ``SPEAR_BTP_WRITE_CHECKPOINT=1`` before importing this
    module (the variable is read once) or call ``spear_amd._btp.forward`` directly to have it written.
"""

from __future__ import annotations

import os

import torch
import torch.library

from spear_amd import _btp

__all__ = ["btp", "btp_log"]

# Fixed by the kernels (interface.py:23-27).
DH = 16
BLK = 16
SUPPORTED_WPB = [4, 8, 16, 32]
WPB_K1_DEFAULT = 8
WPB_K2_DEFAULT = 32


# Read once: the op sits on the hot path of every layer call.
# SPEAR_BTP_PATH=mfma sends the op through the matrix-core kernels (the reference's formulation: a decay matrix
# per block, multiplied on the matrix units) instead of the default fp32 recurrences, forward and backward.
_PATH_MFMA = os.environ.get("SPEAR_BTP_PATH", "") == "mfma"
_FORWARD_FLAGS = (_btp.FLAG_WRITE_CHECKPOINT if os.environ.get("SPEAR_BTP_WRITE_CHECKPOINT", "0") == "1" else 0) | (
    _btp.FLAG_PATH_MFMA if _PATH_MFMA else 0
)


def _forward_impl(
    coeff: torch.Tensor, x: torch.Tensor, y: torch.Tensor, checkpoint: torch.Tensor, k: int, wpb: int
) -> None:
    _btp.load_extension().forward(coeff, x, y, checkpoint, k, wpb, _FORWARD_FLAGS)


def _forward_fake(
    coeff: torch.Tensor, x: torch.Tensor, y: torch.Tensor, checkpoint: torch.Tensor, k: int, wpb: int
) -> None:
    return None


def _backward_impl(
    coeff: torch.Tensor,
    x: torch.Tensor,
    dy: torch.Tensor,
    checkpoint: torch.Tensor,
    dx: torch.Tensor,
    dA: torch.Tensor,
    k: int,
    wpb: int,
) -> None:
    flags = _btp.FLAG_PATH_MFMA if _PATH_MFMA else 0
    _btp.load_extension().backward(coeff, x, dy, checkpoint, dx, dA, k, wpb, flags)


def _backward_fake(
    coeff: torch.Tensor,
    x: torch.Tensor,
    dy: torch.Tensor,
    checkpoint: torch.Tensor,
    dx: torch.Tensor,
    dA: torch.Tensor,
    k: int,
    wpb: int,
) -> None:
    return None


def register_traceable_op(
    lib: torch.library.Library,
    op_name: str,
    op_impl,
    op_fake_impl,
    *,
    mutates_args=None,
    tags=(),
    dispatch_key: str | None = "CUDA",
) -> None:
    """Define ``op_name`` in ``lib`` from the Python signature of ``op_impl``, bind the
    implementation for ``dispatch_key`` and a shape-only fake for tracing (interface.py:36-52).
    On ROCm the device dispatch key is still called "CUDA"."""
    schema = torch.library.infer_schema(op_impl, mutates_args=mutates_args)
    lib.define(op_name + schema, tags=tags)
    lib.impl(op_name, op_impl, dispatch_key=dispatch_key)
    lib._register_fake(op_name, op_fake_impl)


def _forward_log_impl(gate: torch.Tensor, x: torch.Tensor, y: torch.Tensor, k: int) -> None:
    _btp.load_extension().forward_log(gate, x, y, k)


def _forward_log_fake(gate: torch.Tensor, x: torch.Tensor, y: torch.Tensor, k: int) -> None:
    return None


def _backward_log_impl(
    gate: torch.Tensor, x: torch.Tensor, dy: torch.Tensor, dx: torch.Tensor, dgate: torch.Tensor, k: int
) -> None:
    _btp.load_extension().backward_log(gate, x, dy, dx, dgate, k)


def _backward_log_fake(
    gate: torch.Tensor, x: torch.Tensor, dy: torch.Tensor, dx: torch.Tensor, dgate: torch.Tensor, k: int
) -> None:
    return None


lib = torch.library.Library("spear_btp", "DEF")
register_traceable_op(lib, "forward", _forward_impl, _forward_fake, mutates_args=["y", "checkpoint"])
register_traceable_op(lib, "backward", _backward_impl, _backward_fake, mutates_args=["dx", "dA"])
register_traceable_op(lib, "forward_log", _forward_log_impl, _forward_log_fake, mutates_args=["y"])
register_traceable_op(lib, "backward_log", _backward_log_impl, _backward_log_fake, mutates_args=["dx", "dgate"])


def _no_checkpoint(x: torch.Tensor) -> torch.Tensor:
    """The carry checkpoint argument of the forward op: a zero-element placeholder unless the store is on."""
    if _FORWARD_FLAGS & _btp.FLAG_WRITE_CHECKPOINT:
        B, H, _, L = x.shape
        return torch.empty((B, H, L // BLK, DH), device=x.device, dtype=torch.float32)
    return torch.empty((0,), device=x.device, dtype=torch.float32)


class _BTPFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, coeff: torch.Tensor, x: torch.Tensor, k: int, output_dtype: torch.dtype, wpb: int):
        B, H, dh_in, L = x.shape
        assert dh_in == DH, f"Channel dimension must be {DH}"
        assert L % BLK == 0, f"Length L must be multiple of {BLK}"
        assert wpb in SUPPORTED_WPB, f"WPB must be one of {SUPPORTED_WPB}"

        y = torch.empty_like(x, dtype=output_dtype)
        checkpoint = _no_checkpoint(x)
        torch.ops.spear_btp.forward(coeff, x, y, checkpoint, int(k), int(wpb))

        ctx.save_for_backward(coeff, x, checkpoint)
        ctx.k, ctx.wpb, ctx.input_dtype = int(k), int(wpb), x.dtype
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        coeff, x, checkpoint = ctx.saved_tensors
        dy = dy.contiguous()
        dx = torch.empty_like(x, dtype=ctx.input_dtype)
        dA = torch.empty_like(coeff, dtype=torch.float32)
        torch.ops.spear_btp.backward(coeff, x, dy, checkpoint, dx, dA, ctx.k, ctx.wpb)
        return dA, dx, None, None, None


def _plain_eager(*tensors: torch.Tensor) -> bool:
    """True where nothing needs to see the custom ops: ordinary tensors, no torch.compile trace, no dispatch or
    function mode, no functorch transform. Only then may the compiled autograd node stand in for _BTPFunction."""
    try:
        return (
            all(type(t) is torch.Tensor or type(t) is torch.nn.Parameter for t in tensors)
            and not torch.compiler.is_compiling()
            and torch._C._len_torch_dispatch_stack() == 0
            and torch._C._len_torch_function_stack() == 0
            and torch._C._functorch.peek_interpreter_stack() is None
        )
    except AttributeError:  # a PyTorch without these introspection hooks: the Python node is always right
        return False


def btp(
    coeff: torch.Tensor,
    x: torch.Tensor,
    k: int = 2,
    wpb: int | None = None,
    output_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    """Block Two-Pass sliding-window recurrence.

    Args:
        coeff: ``[B, H, L]`` linear-space decay ``a_t``, bf16 or fp16.
        x: ``[B, H, 16, L]`` inputs, same dtype as ``coeff``; ``L`` a multiple of 16.
        k: 1 = block-local only, 2 = local plus the one-hop carry from the previous block.
        wpb: accepted and validated for compatibility (sm90 warps per block); has no effect.
        output_dtype: dtype of the result, ``float32`` (default) or ``x.dtype``.

    Returns:
        ``[B, H, 16, L]`` with ``y_t = sum_{s >= w(t)} (prod_{j=s+1..t} a_j) x_s``.
    """
    out_dtype = output_dtype or torch.float32
    wpb_val = wpb if wpb is not None else (WPB_K2_DEFAULT if k == 2 else WPB_K1_DEFAULT)
    coeff, x = coeff.contiguous(), x.contiguous()
    if not (torch.is_grad_enabled() and (coeff.requires_grad or x.requires_grad)):
        # nothing to differentiate (inference): the op itself, without the autograd node and its bookkeeping
        assert x.dim() == 4 and x.shape[2] == DH, f"Channel dimension must be {DH}"
        assert x.shape[3] % BLK == 0, f"Length L must be multiple of {BLK}"
        assert wpb_val in SUPPORTED_WPB, f"WPB must be one of {SUPPORTED_WPB}"
        y = torch.empty_like(x, dtype=out_dtype)
        torch.ops.spear_btp.forward(coeff, x, y, _no_checkpoint(x), int(k), int(wpb_val))
        return y
    if _plain_eager(coeff, x):
        # the same node, compiled (spear_amd/csrc/btp_torch_ext.cpp): no Python frames between autograd and the kernels
        assert x.dim() == 4 and x.shape[2] == DH, f"Channel dimension must be {DH}"
        assert x.shape[3] % BLK == 0, f"Length L must be multiple of {BLK}"
        assert wpb_val in SUPPORTED_WPB, f"WPB must be one of {SUPPORTED_WPB}"
        if out_dtype not in (torch.float32, x.dtype):  # the binding's own check (csrc/btp/_bindings.cu:33)
            raise RuntimeError("y must be float32 or match x dtype.")
        return _btp.load_extension().btp_autograd(
            coeff, x, int(k), int(wpb_val), out_dtype == torch.float32, _FORWARD_FLAGS,
            _btp.FLAG_PATH_MFMA if _PATH_MFMA else 0,
        )
    return _BTPFunction.apply(coeff, x, k, out_dtype, wpb_val)


class _BTPLogFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate: torch.Tensor, x: torch.Tensor, k: int, output_dtype: torch.dtype):
        B, H, dh_in, L = x.shape
        assert dh_in == DH, f"Channel dimension must be {DH}"
        assert L % BLK == 0, f"Length L must be multiple of {BLK}"
        y = torch.empty_like(x, dtype=output_dtype)
        torch.ops.spear_btp.forward_log(gate, x, y, int(k))
        ctx.save_for_backward(gate, x)
        ctx.k = int(k)
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        gate, x = ctx.saved_tensors
        dx = torch.empty_like(x)
        dgate = torch.empty_like(gate)
        torch.ops.spear_btp.backward_log(gate, x, dy.contiguous(), dx, dgate, ctx.k)
        return dgate, dx, None, None


def btp_log(
    gate: torch.Tensor,
    x: torch.Tensor,
    k: int = 2,
    output_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    """:func:`btp` for callers that hold the decay in log space: ``btp(exp(gate), x)`` with the
    exponential taken in fp32 inside the kernel, and a gradient w.r.t. ``gate`` itself.

    An addition to the reference's API (its op takes the decay already exponentiated and rounded
    to 16 bits). ``gate``: ``[B, H, L]`` float32, ``g_t <= 0`` (e.g. ``-softplus(logit)``);
    ``x``: ``[B, H, 16, L]`` bf16/fp16. Returns ``[B, H, 16, L]`` in ``output_dtype`` (default fp32);
    backward yields ``dgate`` in fp32 and ``dx`` in ``x.dtype``.
    """
    out_dtype = output_dtype or torch.float32
    gate, x = gate.contiguous(), x.contiguous()
    if torch.is_grad_enabled() and (gate.requires_grad or x.requires_grad) and _plain_eager(gate, x):
        # the same node, compiled (spear_amd/csrc/btp_torch_ext.cpp), as btp() has it
        assert x.dim() == 4 and x.shape[2] == DH, f"Channel dimension must be {DH}"
        assert x.shape[3] % BLK == 0, f"Length L must be multiple of {BLK}"
        if out_dtype not in (torch.float32, x.dtype):
            raise RuntimeError("y must be float32 or match x dtype.")
        return _btp.load_extension().btp_log_autograd(gate, x, int(k), out_dtype == torch.float32)
    return _BTPLogFunction.apply(gate, x, k, out_dtype)
