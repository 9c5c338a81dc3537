"""Host shim between torch tensors and the C ABI of ``libspear_btp.so``.

ctypes view of the whole C ABI, used by the tests, the benchmark and the host code of the streaming
and layer paths. The custom ops themselves go through the compiled binding ``spear_amd._btp_ext``
(:func:`load_extension`), which takes the place of the reference's extension module ``spear._btp``
(csrc/btp/_bindings.cu:240-243). Like it, this module exports ``forward(coeff, x, y, checkpoint, k, wpb)`` and
``backward(coeff, x, dy, checkpoint, dx, dA, k, wpb)`` with the same positional arguments, the
same in-place semantics (the caller allocates every output) and the same argument checks and
messages (csrc/btp/_bindings.cu:19-60, raised as ``RuntimeError`` like ``TORCH_CHECK``).

The kernels are enqueued on torch's current stream of the tensors' device and the call returns
without synchronising. There is no fallback: if the library cannot be loaded, every call raises.
"""

from __future__ import annotations

import ctypes
import os
import threading

import torch

__all__ = ["forward", "backward", "forward_log", "backward_log", "mix_forward", "mix_backward", "jagged_prefill", "jagged_step", "library_path", "load_library", "load_extension", "FLAG_WRITE_CHECKPOINT", "FLAG_PATH_MFMA", "FLAG_JAGGED_LOG_A", "FLAG_JAGGED_LOG_R", "FLAG_MIX_QKV_GATE", "FLAG_MIX_F32_RESULTS", "FLAG_DX_F32", "mix_backward_sum_rows", "mix_backward_bias", "mix_step"]

_BF16, _F16, _F32 = 0, 1, 2
FLAG_WRITE_CHECKPOINT = 0x1
FLAG_PATH_MFMA = 0x2
FLAG_JAGGED_LOG_A = 0x4
FLAG_JAGGED_LOG_R = 0x8
FLAG_MIX_QKV_GATE = 0x1
FLAG_MIX_F32_RESULTS = 0x2
FLAG_DX_F32 = 0x10
_ABI_VERSION = 18
_SUPPORTED_WPB = (4, 8, 16, 32)

_lock = threading.Lock()
_lib: ctypes.CDLL | None = None
_load_error: str | None = None


def library_path() -> str:
    return os.environ.get(
        "SPEAR_BTP_LIBRARY",
        os.path.join(os.path.dirname(os.path.abspath(__file__)), "libspear_btp.so"),
    )


def _declare(lib: ctypes.CDLL) -> None:
    vp, ci, cu = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint
    lib.spear_btp_forward.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, cu, vp]
    lib.spear_btp_forward.restype = ci
    lib.spear_btp_backward.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, cu, vp]
    lib.spear_btp_backward.restype = ci
    lib.spear_btp_forward_loggate.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, cu, vp]
    lib.spear_btp_forward_loggate.restype = ci
    lib.spear_btp_backward_loggate.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, ci, cu, vp]
    lib.spear_btp_backward_loggate.restype = ci
    lib.spear_phalanx_mix_forward.argtypes = [vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, cu, vp]
    lib.spear_phalanx_mix_forward.restype = ci
    lib.spear_phalanx_mix_backward.argtypes = [vp] * 9 + [ci, ci, ci, ci, ci, cu, vp]
    lib.spear_phalanx_mix_backward.restype = ci
    lib.spear_phalanx_mix_backward_ex.argtypes = [vp] * 9 + [ci] * 4 + [vp] * 3 + [ctypes.c_longlong, ci, ci, ci, ci, ci, cu, vp]
    lib.spear_phalanx_mix_backward_ex.restype = ci
    lib.spear_phalanx_mix_backward_bias.argtypes = [vp] * 9 + [ci] * 4 + [vp] * 3 + [ci, ci, ci, ci, ci, cu, vp]
    lib.spear_phalanx_mix_backward_bias.restype = ci
    lib.spear_phalanx_mix_backward_sum_rows.argtypes = [ci, ci, ci]
    lib.spear_phalanx_mix_backward_sum_rows.restype = ctypes.c_longlong
    lib.spear_phalanx_mix_prefill.argtypes = [vp, vp, vp, vp, vp, vp, ci, ci, ci, ci, ci, cu, vp]
    lib.spear_phalanx_mix_prefill.restype = ci
    lib.spear_phalanx_mix_step.argtypes = [vp] * 9 + [ci] * 6 + [cu, vp]
    lib.spear_phalanx_mix_step.restype = ci
    lib.spear_jagged_prefill.argtypes = [vp] * 9 + [ci] * 9 + [cu, vp]
    lib.spear_jagged_prefill.restype = ci
    lib.spear_jagged_step.argtypes = [vp] * 11 + [ci] * 8 + [cu, ctypes.c_float, vp]
    lib.spear_jagged_step.restype = ci
    lib.spear_btp_last_error.argtypes = []
    lib.spear_btp_last_error.restype = ctypes.c_char_p
    lib.spear_btp_abi_version.argtypes = []
    lib.spear_btp_abi_version.restype = ci
    lib.spear_btp_copy.argtypes = [vp, vp, ctypes.c_ulonglong, vp]
    lib.spear_btp_copy.restype = ci
    lib.spear_btp_stream_probe.argtypes = [vp, vp, vp, ctypes.c_ulonglong, vp]
    lib.spear_btp_stream_probe.restype = ci
    lib.spear_btp_stream_probe_shape.argtypes = [vp, vp, vp, ctypes.c_ulonglong, ci, vp]
    lib.spear_btp_stream_probe_shape.restype = ci
    lib.spear_btp_stream_probe_mix.argtypes = [ctypes.POINTER(vp), ci, ctypes.POINTER(vp), ci, ctypes.c_ulonglong, ci, vp]
    lib.spear_btp_stream_probe_mix.restype = ci


def load_library() -> ctypes.CDLL:
    """Load (once) and return the native library; raise ``RuntimeError`` if that is impossible."""
    global _lib, _load_error
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = library_path()
        try:
            lib = ctypes.CDLL(path)
            _declare(lib)
            got = lib.spear_btp_abi_version()
            if got != _ABI_VERSION:
                raise OSError(f"ABI version {got}, this package needs {_ABI_VERSION}")
        except (OSError, AttributeError) as exc:
            _load_error = f"{path}: {exc}"
            raise RuntimeError(
                "spear_amd: the HIP BTP library could not be loaded "
                f"({_load_error}). Build it with `python -m spear_amd.csrc.build` (needs hipcc); "
                "there is no CPU fallback for spear_amd.ops.btp.btp."
            ) from exc
        _lib = lib
    return _lib


_ext = None


def load_extension():
    """Import (once) and return ``spear_amd._btp_ext``, the compiled torch binding over the same C ABI
    (``spear_amd/csrc/btp_torch_ext.cpp``): the custom ops call it so that a hot call carries no Python
    argument checks. Raises ``RuntimeError`` if it is not built or does not match this package."""
    global _ext
    if _ext is not None:
        return _ext
    with _lock:
        if _ext is None:
            try:
                import importlib

                ext = importlib.import_module("spear_amd._btp_ext")
            except ImportError as exc:
                raise RuntimeError(
                    f"spear_amd: the compiled torch binding spear_amd/_btp_ext.so could not be imported ({exc}). "
                    "Build it with `python -m spear_amd.csrc.build` (needs hipcc); there is no fallback."
                ) from exc
            if ext.abi_version() != _ABI_VERSION:
                raise RuntimeError(f"spear_amd._btp_ext speaks C ABI {ext.abi_version()}, this package needs {_ABI_VERSION}")
            _ext = ext
    return _ext


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _tag(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return _BF16
    if dtype == torch.float16:
        return _F16
    if dtype == torch.float32:
        return _F32
    return -1


def _check_common(x: torch.Tensor, coeff: torch.Tensor, k: int, wpb: int, wpb_msg: str) -> None:
    _check(x.dim() == 4, "x must be [B, H, 16, L].")
    _check(x.size(2) == 16, "Channel dim (DH) must be 16.")
    _check(k in (1, 2), "k must be 1 or 2.")
    _check(wpb in _SUPPORTED_WPB, f"{wpb_msg}{wpb}")
    _check(coeff.dtype in (torch.float16, torch.bfloat16), "coeff must be float16 or bfloat16.")
    _check(x.dtype == coeff.dtype, "x dtype must match coeff.")


def _check_layout(name: str, t: torch.Tensor, shape: tuple[int, ...]) -> None:
    # The reference reads B*H*L (resp. B*H*16*L) elements without looking at shapes or strides
    # (csrc/btp/_bindings.cu:80-87); a wrong shape there is an out-of-bounds read. Here it raises.
    _check(tuple(t.shape) == shape, f"{name} must have shape {list(shape)}, got {list(t.shape)}.")
    _check(t.is_contiguous(), f"{name} must be contiguous.")


def _row_stride(name: str, t: torch.Tensor, shape: tuple[int, int, int]) -> int:
    """Elements per time step of a ``[B, L, width]`` tensor that is dense or a column block of a wider
    ``[B, L, ld]`` buffer."""
    _check(tuple(t.shape) == shape, f"{name} must have shape {list(shape)}, got {list(t.shape)}.")
    B, L, _ = shape
    ld = t.stride(1) if L > 1 else (t.stride(0) if B > 1 else shape[2])
    _check(t.stride(2) == 1 and (L <= 1 or t.stride(1) == ld) and (B <= 1 or t.stride(0) == L * ld),
           f"{name} must be dense or a column block of a dense [B, L, ld] buffer.")
    return ld


def _raise_native(lib: ctypes.CDLL, rc: int) -> None:
    msg = lib.spear_btp_last_error().decode("utf-8", "replace")
    raise RuntimeError(msg or f"spear_btp call failed with code {rc}")


def _stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def forward(
    coeff: torch.Tensor,
    x: torch.Tensor,
    y: torch.Tensor,
    checkpoint: torch.Tensor,
    k: int,
    wpb: int,
    flags: int = FLAG_WRITE_CHECKPOINT,
) -> None:
    """``y <- btp(coeff, x)`` and ``checkpoint <- carries`` in place (csrc/btp/_bindings.cu:76-150).

    ``flags`` is an extension: drop ``FLAG_WRITE_CHECKPOINT`` to skip the carry store (this
    package's backward recomputes the carries and never reads them).
    """
    _check(coeff.is_cuda and x.is_cuda and y.is_cuda and checkpoint.is_cuda, "All tensors must be CUDA.")
    _check_common(x, coeff, k, wpb, "Unsupported WPB value: ")
    _check(y.dtype == torch.float32 or y.dtype == x.dtype, "y must be float32 or match x dtype.")
    _check(checkpoint.dtype == torch.float32, "checkpoint must be float32.")
    B, H, _, L = x.shape
    _check(L % 16 == 0, "Length L must be multiple of 16")
    _check_layout("coeff", coeff, (B, H, L))
    _check_layout("x", x, (B, H, 16, L))
    _check_layout("y", y, (B, H, 16, L))
    if flags & FLAG_WRITE_CHECKPOINT or checkpoint.numel() != 0:  # a zero-element placeholder when it is not stored
        _check_layout("checkpoint", checkpoint, (B, H, L // 16, 16))
    _check(coeff.device == x.device == y.device == checkpoint.device, "All tensors must be on the same device.")

    lib = load_library()
    with torch.cuda.device(x.device):
        rc = lib.spear_btp_forward(
            coeff.data_ptr(), x.data_ptr(), y.data_ptr(), checkpoint.data_ptr(),
            B, H, L, int(k), _tag(x.dtype), _tag(y.dtype), int(flags), _stream_ptr(x.device),
        )
    if rc != 0:
        _raise_native(lib, rc)


def backward(
    coeff: torch.Tensor,
    x: torch.Tensor,
    dy: torch.Tensor,
    checkpoint: torch.Tensor,
    dx: torch.Tensor,
    dA: torch.Tensor,
    k: int,
    wpb: int,
    flags: int = 0,
) -> None:
    """``dx, dA <- vjp of btp at (coeff, x) applied to dy``, in place (csrc/btp/_bindings.cu:152-229).

    Every element of ``dA`` is written, so it need not arrive zero-filled. ``checkpoint`` is
    accepted for signature compatibility and not read. ``flags`` is an extension: with ``FLAG_DX_F32``
    ``dx`` is a float32 tensor and receives the kernel's fp32 values unrounded (fp32 check mode).
    """
    _check(
        coeff.is_cuda and x.is_cuda and dy.is_cuda and checkpoint.is_cuda,
        "coeff, x, dy, checkpoint must be CUDA.",
    )
    _check(dx.is_cuda and dA.is_cuda, "dx and dA must be CUDA.")
    _check_common(x, coeff, k, wpb, "Unsupported WPB value for backward: ")
    if flags & FLAG_DX_F32:
        _check(dx.dtype == torch.float32, "dx must be float32 in the fp32 check mode.")
    else:
        _check(dx.dtype == x.dtype, "dx dtype must match x.")
    _check(dA.dtype == torch.float32, "dA must be float32.")
    _check(dy.dtype == torch.float32 or dy.dtype == x.dtype, "dy must be float32 or match x dtype.")
    B, H, _, L = x.shape
    _check(L % 16 == 0, "Length L must be multiple of 16")
    _check_layout("coeff", coeff, (B, H, L))
    _check_layout("x", x, (B, H, 16, L))
    _check_layout("dy", dy, (B, H, 16, L))
    _check_layout("dx", dx, (B, H, 16, L))
    _check_layout("dA", dA, (B, H, L))
    _check(coeff.device == x.device == dy.device == dx.device == dA.device, "All tensors must be on the same device.")

    lib = load_library()
    with torch.cuda.device(x.device):
        rc = lib.spear_btp_backward(
            coeff.data_ptr(), x.data_ptr(), dy.data_ptr(), checkpoint.data_ptr(), dx.data_ptr(), dA.data_ptr(),
            B, H, L, int(k), _tag(x.dtype), _tag(dy.dtype), int(flags), _stream_ptr(x.device),
        )
    if rc != 0:
        _raise_native(lib, rc)


def _check_log_common(gate: torch.Tensor, x: torch.Tensor, k: int) -> tuple[int, int, int]:
    _check(gate.is_cuda and x.is_cuda, "All tensors must be CUDA.")
    _check(x.dim() == 4, "x must be [B, H, 16, L].")
    _check(x.size(2) == 16, "Channel dim (DH) must be 16.")
    _check(k in (1, 2), "k must be 1 or 2.")
    _check(gate.dtype == torch.float32, "gate must be float32.")
    _check(x.dtype in (torch.float16, torch.bfloat16), "x must be float16 or bfloat16.")
    B, H, _, L = x.shape
    _check(L % 16 == 0, "Length L must be multiple of 16")
    _check_layout("gate", gate, (B, H, L))
    _check_layout("x", x, (B, H, 16, L))
    return B, H, L


def forward_log(gate: torch.Tensor, x: torch.Tensor, y: torch.Tensor, k: int) -> None:
    """``y <- btp(exp(gate), x)`` with the exponential taken in fp32 inside the kernel. ``gate`` is
    the fp32 log-space decay ``[B, H, L]``. No counterpart in the reference's extension module."""
    B, H, L = _check_log_common(gate, x, k)
    _check(y.is_cuda, "All tensors must be CUDA.")
    _check(y.dtype == torch.float32 or y.dtype == x.dtype, "y must be float32 or match x dtype.")
    _check_layout("y", y, (B, H, 16, L))
    _check(gate.device == x.device == y.device, "All tensors must be on the same device.")
    lib = load_library()
    with torch.cuda.device(x.device):
        rc = lib.spear_btp_forward_loggate(
            gate.data_ptr(), x.data_ptr(), y.data_ptr(), None, B, H, L, int(k), _tag(x.dtype), _tag(y.dtype), 0,
            _stream_ptr(x.device),
        )
    if rc != 0:
        _raise_native(lib, rc)


def backward_log(
    gate: torch.Tensor, x: torch.Tensor, dy: torch.Tensor, dx: torch.Tensor, dgate: torch.Tensor, k: int
) -> None:
    """``dx, dgate <- vjp of btp(exp(gate), x)``; ``dgate`` is the gradient w.r.t. the log-space gate.
    A float32 ``dx`` selects the fp32 check mode (``SPEAR_BTP_DX_F32``)."""
    B, H, L = _check_log_common(gate, x, k)
    _check(dy.is_cuda and dx.is_cuda and dgate.is_cuda, "All tensors must be CUDA.")
    _check(dx.dtype in (x.dtype, torch.float32), "dx must be float32 or match x dtype.")
    _check(dgate.dtype == torch.float32, "dgate must be float32.")
    _check(dy.dtype == torch.float32 or dy.dtype == x.dtype, "dy must be float32 or match x dtype.")
    _check_layout("dy", dy, (B, H, 16, L))
    _check_layout("dx", dx, (B, H, 16, L))
    _check_layout("dgate", dgate, (B, H, L))
    _check(gate.device == x.device == dy.device == dx.device == dgate.device, "All tensors must be on the same device.")
    lib = load_library()
    with torch.cuda.device(x.device):
        rc = lib.spear_btp_backward_loggate(
            gate.data_ptr(), x.data_ptr(), dy.data_ptr(), dx.data_ptr(), dgate.data_ptr(), B, H, L, int(k),
            _tag(x.dtype), _tag(dy.dtype), FLAG_DX_F32 if dx.dtype == torch.float32 else 0, _stream_ptr(x.device),
        )
    if rc != 0:
        _raise_native(lib, rc)


def mix_forward(
    a_logit: torch.Tensor,
    b_logit: torch.Tensor,
    c: torch.Tensor,
    v: torch.Tensor,
    out: torch.Tensor,
    heads: int,
    kv_heads: int,
    qkv_gate: bool = False,
    c_prev_tail: torch.Tensor | None = None,
) -> None:
    """``out <- btp(sigmoid(a_logit), sigmoid(b_logit) * v) * c + v`` with every operand in the
    layer's ``[B, L, features]`` layout (see ``spear_phalanx_mix_forward`` in the C header).
    ``qkv_gate``: ``a_logit`` is an fp32 log-decay gate, ``b_logit`` is k, ``c`` is q:
    ``out <- c * btp(exp(a_logit), b_logit * v) + v`` (``SPEAR_MIX_QKV_GATE``). ``c_prev_tail``: fp32
    ``[B, heads, 16]`` that receives the terminal local state of every row's last block, the hand-over state
    for decoding after this prompt (``spear_phalanx_mix_prefill``)."""
    _check(all(t.is_cuda for t in (a_logit, b_logit, c, v, out)), "All tensors must be CUDA.")
    _check(v.dim() == 3, "v must be [B, L, heads * 16].")
    B, L, F = v.shape
    _check(F == heads * 16, "v must be [B, L, heads * 16].")
    _check(heads > 0 and kv_heads > 0 and heads % kv_heads == 0, "heads must be divisible by kv_heads.")
    _check(v.dtype in (torch.float16, torch.bfloat16), "tensors must be float16 or bfloat16.")
    _check(b_logit.dtype == c.dtype == v.dtype, "all tensors must share one dtype.")
    _check(out.dtype in (v.dtype, torch.float32), "out must be float32 (fp32 check mode) or match v dtype.")
    f32 = out.dtype == torch.float32
    if qkv_gate:
        _check(a_logit.dtype == torch.float32, "the log-decay gate must be float32.")
    else:
        _check(a_logit.dtype == v.dtype, "all tensors must share one dtype.")
    _check(L % 16 == 0, "Length L must be multiple of 16")
    _check_layout("a_logit", a_logit, (B, L, heads))
    _check_layout("b_logit", b_logit, (B, L, kv_heads * 16))
    _check_layout("c", c, (B, L, kv_heads * 16))
    _check_layout("v", v, (B, L, F))
    _check_layout("out", out, (B, L, F))
    _check(len({t.device for t in (a_logit, b_logit, c, v, out)}) == 1, "All tensors must be on the same device.")
    if c_prev_tail is not None:
        _check(c_prev_tail.is_cuda and c_prev_tail.device == v.device and c_prev_tail.dtype == torch.float32,
               "c_prev_tail must be float32 on v's device.")
        _check_layout("c_prev_tail", c_prev_tail, (B, heads, 16))
    lib = load_library()
    with torch.cuda.device(v.device):
        rc = lib.spear_phalanx_mix_prefill(
            a_logit.data_ptr(), b_logit.data_ptr(), c.data_ptr(), v.data_ptr(), out.data_ptr(), _ptr(c_prev_tail),
            B, L, heads, kv_heads, _tag(v.dtype),
            (FLAG_MIX_QKV_GATE if qkv_gate else 0) | (FLAG_MIX_F32_RESULTS if f32 else 0),
            _stream_ptr(v.device),
        )
    if rc != 0:
        _raise_native(lib, rc)


def mix_backward_sum_rows(B: int, L: int, heads: int) -> int:
    """Rows of the partial-sum arrays :func:`mix_backward` fills for this shape: one per (batch row, tile of 64
    time steps)."""
    return int(load_library().spear_phalanx_mix_backward_sum_rows(B, L, heads))


def mix_backward(
    a_logit: torch.Tensor,
    b_logit: torch.Tensor,
    c: torch.Tensor,
    v: torch.Tensor,
    dout: torch.Tensor,
    da_logit: torch.Tensor,
    db_logit: torch.Tensor,
    dc: torch.Tensor,
    dv: torch.Tensor,
    heads: int,
    kv_heads: int,
    sums: tuple[torch.Tensor, torch.Tensor, torch.Tensor] | None = None,
    qkv_gate: bool = False,
) -> None:
    """Gradients of :func:`mix_forward`, written in place, for any ``heads % kv_heads == 0``
    (see ``spear_phalanx_mix_backward`` in the C header). ``sums``: three fp32 tensors
    ``[mix_backward_sum_rows(B, L, heads), heads | kv_heads*16 | kv_heads*16]`` that receive the column sums of
    ``da_logit``, ``db_logit`` and ``dc`` per (batch row, tile of 64 time steps). The four gradient tensors may be
    column blocks of one wider ``[B, L, ld]`` buffer (``spear_phalanx_mix_backward_ex``). ``qkv_gate`` as in
    :func:`mix_forward`; ``da_logit`` is then the fp32 gradient of the gate. Float32 ``db_logit, dc, dv`` (and
    ``da_logit``) select the fp32 check mode (``SPEAR_MIX_F32_RESULTS``)."""
    tensors = (a_logit, b_logit, c, v, dout, da_logit, db_logit, dc, dv)
    _check(all(t.is_cuda for t in tensors), "All tensors must be CUDA.")
    _check(v.dim() == 3, "v must be [B, L, heads * 16].")
    B, L, F = v.shape
    _check(F == heads * 16, "v must be [B, L, heads * 16].")
    _check(heads > 0 and kv_heads > 0 and heads % kv_heads == 0, "heads must be divisible by kv_heads.")
    _check(v.dtype in (torch.float16, torch.bfloat16), "tensors must be float16 or bfloat16.")
    f32 = dv.dtype == torch.float32  # fp32 check mode: the four gradients are stored unrounded
    _check(all(t.dtype == v.dtype for t in (b_logit, c, dout)), "all tensors must share one dtype.")
    _check(all(t.dtype == dv.dtype for t in (db_logit, dc)) and dv.dtype in (v.dtype, torch.float32),
           "db_logit, dc and dv must all be float32 (fp32 check mode) or all match v dtype.")
    _check(a_logit.dtype == (torch.float32 if qkv_gate else v.dtype),
           "the log-decay gate must be float32." if qkv_gate else "all tensors must share one dtype.")
    _check(da_logit.dtype == (torch.float32 if (qkv_gate or f32) else v.dtype),
           "the gradient of the gate must be float32." if (qkv_gate or f32) else "all tensors must share one dtype.")
    _check(sums is None or not f32, "column sums are not available in the fp32 check mode.")
    _check(sums is None or not qkv_gate, "column sums belong to the layer form, not to qkv_gate.")
    _check(L % 16 == 0, "Length L must be multiple of 16")
    Fkv = kv_heads * 16
    for name, t, shape in (
        ("a_logit", a_logit, (B, L, heads)), ("b_logit", b_logit, (B, L, Fkv)), ("c", c, (B, L, Fkv)),
        ("v", v, (B, L, F)), ("dout", dout, (B, L, F)),
    ):
        _check_layout(name, t, shape)
    lds = [_row_stride(name, t, (B, L, width)) for name, t, width in
           (("da_logit", da_logit, heads), ("db_logit", db_logit, Fkv), ("dc", dc, Fkv), ("dv", dv, F))]
    _check(len({t.device for t in tensors}) == 1, "All tensors must be on the same device.")
    lib = load_library()
    rows = 0
    if sums is not None:
        rows = mix_backward_sum_rows(B, L, heads)
        for name, t, width in (("sum_da", sums[0], heads), ("sum_db", sums[1], Fkv), ("sum_dc", sums[2], Fkv)):
            _check(t.is_cuda and t.device == v.device and t.dtype == torch.float32, f"{name} must be float32 on v's device.")
            _check_layout(name, t, (rows, width))
    sum_ptrs = [t.data_ptr() for t in sums] if rows > 0 else [None, None, None]
    with torch.cuda.device(v.device):
        rc = lib.spear_phalanx_mix_backward_ex(
            a_logit.data_ptr(), b_logit.data_ptr(), c.data_ptr(), v.data_ptr(), dout.data_ptr(),
            da_logit.data_ptr(), db_logit.data_ptr(), dc.data_ptr(), dv.data_ptr(), *lds,
            *sum_ptrs, rows,
            B, L, heads, kv_heads, _tag(v.dtype),
            (FLAG_MIX_QKV_GATE if qkv_gate else 0) | (FLAG_MIX_F32_RESULTS if f32 else 0),
            _stream_ptr(v.device),
        )
    if rc != 0:
        _raise_native(lib, rc)


def mix_backward_bias(
    a_logit: torch.Tensor,
    b_logit: torch.Tensor,
    c: torch.Tensor,
    v: torch.Tensor,
    dout: torch.Tensor,
    da_logit: torch.Tensor,
    db_logit: torch.Tensor,
    dc: torch.Tensor,
    dv: torch.Tensor,
    bias: tuple[torch.Tensor, torch.Tensor, torch.Tensor],
    heads: int,
    kv_heads: int,
) -> None:
    """:func:`mix_backward` plus the finished column sums of ``da_logit``, ``db_logit`` and ``dc`` over batch
    and time in ``bias`` (fp32 ``[heads]``, ``[kv_heads*16]``, ``[kv_heads*16]``), with no device memory
    allocated anywhere on the way: the partial sums pass through an array the library holds statically
    (``spear_phalanx_mix_backward_bias`` in the C header; shapes beyond its size raise). Calls on one GPU
    must not overlap in time."""
    tensors = (a_logit, b_logit, c, v, dout, da_logit, db_logit, dc, dv, *bias)
    _check(all(t.is_cuda for t in tensors), "All tensors must be CUDA.")
    _check(len({t.device for t in tensors}) == 1, "All tensors must be on the same device.")
    _check(v.dim() == 3, "v must be [B, L, heads * 16].")
    B, L, F = v.shape
    _check(F == heads * 16, "v must be [B, L, heads * 16].")
    _check(kv_heads > 0 and heads % kv_heads == 0, "heads must be divisible by kv_heads.")
    _check(v.dtype in (torch.float16, torch.bfloat16), "tensors must be float16 or bfloat16.")
    _check(all(t.dtype == v.dtype for t in tensors[:9]), "all tensors must share one dtype.")
    Fkv = kv_heads * 16
    for name, t, shape in (
        ("a_logit", a_logit, (B, L, heads)), ("b_logit", b_logit, (B, L, Fkv)), ("c", c, (B, L, Fkv)),
        ("v", v, (B, L, F)), ("dout", dout, (B, L, F)),
    ):
        _check_layout(name, t, shape)
    lds = [_row_stride(name, t, (B, L, width)) for name, t, width in
           (("da_logit", da_logit, heads), ("db_logit", db_logit, Fkv), ("dc", dc, Fkv), ("dv", dv, F))]
    for name, t, width in (("bias_da", bias[0], heads), ("bias_db", bias[1], Fkv), ("bias_dc", bias[2], Fkv)):
        _check(t.dtype == torch.float32, f"{name} must be float32.")
        _check_layout(name, t, (width,))
    lib = load_library()
    with torch.cuda.device(v.device):
        rc = lib.spear_phalanx_mix_backward_bias(
            a_logit.data_ptr(), b_logit.data_ptr(), c.data_ptr(), v.data_ptr(), dout.data_ptr(),
            da_logit.data_ptr(), db_logit.data_ptr(), dc.data_ptr(), dv.data_ptr(), *lds,
            bias[0].data_ptr(), bias[1].data_ptr(), bias[2].data_ptr(),
            B, L, heads, kv_heads, _tag(v.dtype), 0, _stream_ptr(v.device),
        )
    if rc != 0:
        _raise_native(lib, rc)


def mix_step(
    a_logit: torch.Tensor,
    b_logit: torch.Tensor,
    c: torch.Tensor,
    v: torch.Tensor,
    out: torch.Tensor,
    h: torch.Tensor,
    r: torch.Tensor,
    c_prev: torch.Tensor,
    pos: torch.Tensor | None,
    boundary: bool,
    block_len: int,
    heads: int,
    kv_heads: int,
) -> None:
    """One decode token of the mixing stage on the projections' ``[B, features]`` outputs; the fp32 state
    ``h, r, c_prev`` is updated in place (see ``spear_phalanx_mix_step`` in the C header). ``pos``: int32 ``[B]``
    positions inside the block (advanced by the call) or ``None`` to let ``boundary`` decide for all rows."""
    tensors = [a_logit, b_logit, c, v, out, h, r, c_prev] + ([pos] if pos is not None else [])
    _check(all(t.is_cuda for t in tensors), "All tensors must be CUDA.")
    _check(len({t.device for t in tensors}) == 1, "All tensors must be on the same device.")
    _check(v.dim() == 2 and v.shape[1] == heads * 16, "v must be [B, heads * 16].")
    B = v.shape[0]
    _check(kv_heads > 0 and heads % kv_heads == 0, "heads must be divisible by kv_heads.")
    _check(v.dtype in (torch.float16, torch.bfloat16), "tensors must be float16 or bfloat16.")
    _check(all(t.dtype == v.dtype for t in (a_logit, b_logit, c, out)), "all tensors must share one dtype.")
    _check(all(t.dtype == torch.float32 for t in (h, r, c_prev)), "the state must be float32.")
    _check_layout("a_logit", a_logit, (B, heads))
    _check_layout("b_logit", b_logit, (B, kv_heads * 16))
    _check_layout("c", c, (B, kv_heads * 16))
    _check_layout("v", v, (B, heads * 16))
    _check_layout("out", out, (B, heads * 16))
    _check_layout("h", h, (B, heads, 16))
    _check_layout("c_prev", c_prev, (B, heads, 16))
    _check_layout("r", r, (B, heads))
    if pos is not None:
        _check(pos.dtype == torch.int32, "pos must be int32.")
        _check_layout("pos", pos, (B,))
    lib = load_library()
    with torch.cuda.device(v.device):
        rc = lib.spear_phalanx_mix_step(
            a_logit.data_ptr(), b_logit.data_ptr(), c.data_ptr(), v.data_ptr(), out.data_ptr(), h.data_ptr(),
            r.data_ptr(), c_prev.data_ptr(), _ptr(pos), int(bool(boundary)), int(block_len), B, heads, kv_heads,
            _tag(v.dtype), 0, _stream_ptr(v.device),
        )
    if rc != 0:
        _raise_native(lib, rc)


def _ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def jagged_prefill(
    a: torch.Tensor,
    x: torch.Tensor,
    c: torch.Tensor | None,
    v: torch.Tensor | None,
    carry_init: torch.Tensor | None,
    y: torch.Tensor,
    h_tail: torch.Tensor | None,
    r_tail: torch.Tensor | None,
    c_prev_tail: torch.Tensor | None,
    block_len: int,
    log_a: bool,
) -> None:
    """``y <- (block-local scan of (a, x) + one-hop carry) * c + v`` on ``[B, H, D, L]`` tensors and, if
    the three state tensors are given, the state after the last step (see ``spear_jagged_prefill`` in
    the C header). Everything is written in place; nothing is allocated."""
    given = [t for t in (a, x, c, v, carry_init, y, h_tail, r_tail, c_prev_tail) if t is not None]
    _check(all(t.is_cuda for t in given), "All tensors must be CUDA.")
    _check(len({t.device for t in given}) == 1, "All tensors must be on the same device.")
    _check(x.dim() == 4, "x must be [B, H, D, L].")
    B, H, D, L = x.shape
    _check(_tag(x.dtype) >= 0, "x must be float32, float16 or bfloat16.")
    _check(a.dtype == x.dtype or a.dtype == torch.float32, "a must be float32 or match x dtype.")
    _check((c is None) == (v is None), "c and v must be given together.")
    _check(block_len > 0, "block_len must be positive.")
    _check_layout("a", a, (B, H, L))
    _check_layout("x", x, (B, H, D, L))
    _check_layout("y", y, (B, H, D, L))
    _check(y.dtype == x.dtype, "y dtype must match x.")
    for name, t in (("c", c), ("v", v)):
        if t is not None:
            _check_layout(name, t, (B, H, D, L))
            _check(t.dtype == x.dtype, f"{name} dtype must match x.")
    state = (h_tail, r_tail, c_prev_tail)
    _check(all(t is None for t in state) or all(t is not None for t in state), "state tensors must be given together.")
    state_dtype = x.dtype
    if h_tail is not None:
        _check_layout("h_tail", h_tail, (B, H, D))
        _check_layout("c_prev_tail", c_prev_tail, (B, H, D))
        _check_layout("r_tail", r_tail, (B, H))
        _check(h_tail.dtype == c_prev_tail.dtype, "h_tail and c_prev_tail must share a dtype.")
        _check(h_tail.dtype in (x.dtype, torch.float32), "the state must be float32 or match x dtype.")
        _check(_tag(r_tail.dtype) >= 0, "r_tail must be float32, float16 or bfloat16.")
        state_dtype = h_tail.dtype
    if carry_init is not None:
        _check_layout("carry_init", carry_init, (B, H, D))
        _check(h_tail is None or carry_init.dtype == state_dtype, "carry_init must have the state's dtype.")
        _check(carry_init.dtype in (x.dtype, torch.float32), "carry_init must be float32 or match x dtype.")
        state_dtype = carry_init.dtype
    lib = load_library()
    with torch.cuda.device(x.device):
        rc = lib.spear_jagged_prefill(
            a.data_ptr(), x.data_ptr(), _ptr(c), _ptr(v), _ptr(carry_init), y.data_ptr(),
            _ptr(h_tail), _ptr(r_tail), _ptr(c_prev_tail), B, H, D, L, int(block_len),
            _tag(a.dtype), _tag(x.dtype), _tag(state_dtype), _tag(r_tail.dtype) if r_tail is not None else _F32,
            FLAG_JAGGED_LOG_A if log_a else 0, _stream_ptr(x.device),
        )
    if rc != 0:
        _raise_native(lib, rc)


def jagged_step(
    a_t: torch.Tensor,
    x_t: torch.Tensor,
    c_t: torch.Tensor | None,
    v_t: torch.Tensor | None,
    y_t: torch.Tensor,
    h_in: torch.Tensor,
    r_in: torch.Tensor,
    c_prev_in: torch.Tensor,
    h_out: torch.Tensor,
    r_out: torch.Tensor,
    c_prev_out: torch.Tensor | None,
    boundary: bool,
    log_a: bool,
    log_r: bool,
    tiny: float,
) -> None:
    """One decode token for every (batch, head) (see ``spear_jagged_step`` in the C header). Outputs
    are written in place; each ``*_out`` may be the same tensor as its ``*_in``."""
    given = [t for t in (a_t, x_t, c_t, v_t, y_t, h_in, r_in, c_prev_in, h_out, r_out, c_prev_out) if t is not None]
    _check(all(t.is_cuda for t in given), "All tensors must be CUDA.")
    _check(len({t.device for t in given}) == 1, "All tensors must be on the same device.")
    _check(x_t.dim() == 3, "x_t must be [B, H, D].")
    B, H, D = x_t.shape
    _check(_tag(x_t.dtype) >= 0 and _tag(a_t.dtype) >= 0, "tensors must be float32, float16 or bfloat16.")
    _check((c_t is None) == (v_t is None), "c_t and v_t must be given together.")
    _check(not boundary or c_prev_out is not None, "c_prev_out is required at a block boundary.")
    _check_layout("a_t", a_t, (B, H))
    for name, t in (("x_t", x_t), ("c_t", c_t), ("v_t", v_t), ("y_t", y_t)):
        if t is not None:
            _check_layout(name, t, (B, H, D))
            _check(t.dtype == x_t.dtype, f"{name} dtype must match x_t.")
    for name, t in (("h_in", h_in), ("c_prev_in", c_prev_in), ("h_out", h_out), ("c_prev_out", c_prev_out)):
        if t is not None:
            _check_layout(name, t, (B, H, D))
            _check(t.dtype == h_in.dtype, "state tensors must share a dtype.")
    _check(h_in.dtype in (x_t.dtype, torch.float32), "the state must be float32 or match x_t dtype.")
    _check_layout("r_in", r_in, (B, H))
    _check_layout("r_out", r_out, (B, H))
    _check(r_in.dtype == r_out.dtype and _tag(r_in.dtype) >= 0, "r_in and r_out must share a float dtype.")
    flags = (FLAG_JAGGED_LOG_A if log_a else 0) | (FLAG_JAGGED_LOG_R if log_r else 0)
    lib = load_library()
    with torch.cuda.device(x_t.device):
        rc = lib.spear_jagged_step(
            a_t.data_ptr(), x_t.data_ptr(), _ptr(c_t), _ptr(v_t), y_t.data_ptr(), h_in.data_ptr(), r_in.data_ptr(),
            c_prev_in.data_ptr(), h_out.data_ptr(), r_out.data_ptr(), _ptr(c_prev_out), B, H, D, int(bool(boundary)),
            _tag(a_t.dtype), _tag(x_t.dtype), _tag(h_in.dtype), _tag(r_in.dtype), flags, float(tiny),
            _stream_ptr(x_t.device),
        )
    if rc != 0:
        _raise_native(lib, rc)
