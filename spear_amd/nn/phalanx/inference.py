"""Streaming inference for the block two-pass recurrence on MI355X: prompt prefill with the state
hand-over, and token-by-token decoding.

Drop-in for the reference's ``spear.nn.phalanx.inference`` (spear/nn/phalanx/inference.py): the
same five public names with the same arguments and return values,

    jagged_band_infer_sequential(u, a, block_len, *, use_log_a=False, carry_init=None) -> y      :36-92
    JaggedBandState(B, H, D, block_len, device=None, dtype=None).step(a_t, u_t, *, use_log_a)    :95-140
    JagState(h_loc, r_pref, c_prev_loc, i, block_len, use_log_r=False, log_r_pref=None)          :142-175
    step_jagged(A_t, X_t, C_t, V_t, state, *, use_log_a=False) -> (y_t, JagState)                :178-278
    parallel_jagged(A, X, C, V, *, block_len, use_log_a=False) -> (Y, JagState)                  :281-360

but every loop over time, blocks and tokens is a HIP kernel call (``spear_jagged_prefill`` /
``spear_jagged_step`` of the native library) instead of a chain of PyTorch ops. Tensors must live
on the GPU; there is no CPU path.

What differs from the reference, none of it in the values beyond rounding:
  * arithmetic is fp32 inside the kernels whatever the storage dtype, and results are rounded
    once when stored (the reference rounds after every PyTorch op in the tensors' dtype);
  * outputs have the dtype of the driving term (``u`` / ``X_t`` / ``X``); the reference's type
    promotion gives the same dtype whenever all operands share one;
  * ``step_jagged(..., inplace=True)`` and ``parallel_jagged(..., state_dtype=...)`` are additions:
    the first updates the state's own tensors instead of allocating new ones each token, the
    second keeps the hand-over state in fp32 when the tensors are 16-bit.

Additions for decoding with the whole layer (no counterpart in the reference, whose step function takes
gated, kv-expanded ``[B, H, D]`` operands): ``phalanx_step(layer, x_t, state)`` runs one token through a
``Phalanx`` layer -- four projections, ONE kernel for gates + recurrence step + ``* C + V`` on the projections'
``[B, features]`` outputs (``spear_phalanx_mix_step``), output projection -- with the block position kept on the
device, so that the step records into one HIP graph that serves every token; ``phalanx_prefill`` runs a prompt
through the layer (fused forward kernel, which also leaves the hand-over state) and returns the state to continue from.

The state ``parallel_jagged`` returns for a prompt whose length is a multiple of ``block_len``
follows the reference as written (inference.py:327-341): ``h_loc`` is the last block's terminal
local state, not zero, so a decode step taken from that state counts it twice. Prompts of any
other length hand over a state from which decoding continues the prefill exactly.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from spear_amd import _btp

__all__ = [
    "jagged_band_infer_sequential",
    "JaggedBandState",
    "JagState",
    "step_jagged",
    "parallel_jagged",
    "PhalanxStepState",
    "phalanx_prefill",
    "phalanx_step",
]


def _need_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "spear_amd.nn.phalanx.inference runs HIP kernels only: tensors must be on a GPU device "
                f"(got a tensor on {t.device})."
            )


@torch.no_grad()
def jagged_band_infer_sequential(
    u: torch.Tensor,  # (B, H, D, N)
    a: torch.Tensor,  # (B, H, N)  (raw gates unless use_log_a=True)
    block_len: int,
    *,
    use_log_a: bool = False,
    carry_init: torch.Tensor | None = None,  # (B, H, D), optional prior local carry for block -1
) -> torch.Tensor:
    """``y_t = y_loc_t + r_pref_t * c_prev_loc``: block-local scan from zero plus the previous
    block's frozen terminal local state times the inclusive in-block gate product
    (inference.py:36-92). Returns ``y`` with the shape and dtype of ``u``."""
    assert u.ndim == 4 and a.ndim == 3, "u: (B,H,D,N), a: (B,H,N)"
    B, H, D, N = u.shape
    assert a.shape == (B, H, N)
    _need_gpu(u, a, carry_init)
    u = u.contiguous()
    y = torch.empty_like(u)
    carry = None if carry_init is None else carry_init.to(device=u.device, dtype=u.dtype).contiguous()
    a = a.contiguous()
    if a.dtype != u.dtype and a.dtype != torch.float32:
        a = a.float()
    _btp.jagged_prefill(a, u, None, None, carry, y, None, None, None, block_len, use_log_a)
    return y


class JaggedBandState:
    """Streaming state for token-by-token inference (inference.py:95-140).

    ``step()`` implements ``y_loc <- a_t * y_loc + u_t``, ``r_pref <- a_t * r_pref`` (inclusive),
    ``y_t <- y_loc + r_pref * c_prev_loc`` and snapshots ``c_prev_loc`` at block boundaries. The
    state tensors are updated in place by one kernel per token.
    """

    def __init__(self, B: int, H: int, D: int, block_len: int, device=None, dtype=None):
        device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if device.type != "cuda":
            raise RuntimeError("JaggedBandState runs HIP kernels only: device must be a GPU.")
        self.block_len = block_len
        self.y_loc = torch.zeros(B, H, D, device=device, dtype=dtype)
        self.r_pref = torch.ones(B, H, 1, device=device, dtype=dtype)
        self.c_prev_loc = torch.zeros(B, H, D, device=device, dtype=dtype)
        self.i = 0

    @torch.no_grad()
    def reset_block(self):
        self.y_loc.zero_()
        self.r_pref.fill_(1.0)
        self.i = 0

    @torch.no_grad()
    def step(self, a_t: torch.Tensor, u_t: torch.Tensor, *, use_log_a: bool = False) -> torch.Tensor:
        """a_t: (B,H) or (B,H,1), raw or log per ``use_log_a``; u_t: (B,H,D). Returns y_t (B,H,D)."""
        _need_gpu(a_t, u_t)
        if a_t.ndim == 3:
            a_t = a_t.squeeze(-1)
        u_t = u_t.contiguous()
        y_t = torch.empty_like(u_t)
        boundary = self.i + 1 == self.block_len
        r = self.r_pref.view(self.r_pref.shape[0], self.r_pref.shape[1])
        _btp.jagged_step(
            a_t.contiguous(), u_t, None, None, y_t, self.y_loc, r, self.c_prev_loc, self.y_loc, r, self.c_prev_loc,
            boundary, use_log_a, False, 0.0,
        )
        self.i = 0 if boundary else self.i + 1
        return y_t


@dataclass
class JagState:
    """Minimal streaming state (inference.py:142-175).

    - h_loc: (B, H, D)       block-local accumulator
    - r_pref: (B, H)         inclusive gate product within the current block (None in log space)
    - c_prev_loc: (B, H, D)  snapshot of the previous block's terminal local state
    - i: int                 in-block index of the next token (0..block_len-1)
    - block_len: int         block length used during prefill
    - use_log_r: bool        accumulate the gate product in log space
    - log_r_pref: (B, H)     log of the gate product (None unless in log space)
    """

    h_loc: torch.Tensor
    r_pref: torch.Tensor | None
    c_prev_loc: torch.Tensor
    i: int
    block_len: int
    use_log_r: bool = False
    log_r_pref: torch.Tensor | None = None

    def clone_detached(self) -> "JagState":
        return JagState(
            h_loc=self.h_loc.clone(),
            r_pref=None if self.r_pref is None else self.r_pref.clone(),
            c_prev_loc=self.c_prev_loc.clone(),
            i=int(self.i),
            block_len=int(self.block_len),
            use_log_r=bool(self.use_log_r),
            log_r_pref=None if self.log_r_pref is None else self.log_r_pref.clone(),
        )


@torch.no_grad()
def step_jagged(
    A_t: torch.Tensor,  # (B, H)      a_t if use_log_a=False, log(a_t) if True
    X_t: torch.Tensor,  # (B, H, D)   driving term (e.g., B_t * V_t)
    C_t: torch.Tensor,  # (B, H, D)
    V_t: torch.Tensor,  # (B, H, D)
    state: JagState,
    *,
    use_log_a: bool = False,
    inplace: bool = False,
) -> tuple[torch.Tensor, JagState]:
    """One decode token (inference.py:178-278): ``h = a_t * h_loc + X_t``, ``r = a_t * r_pref`` (or
    its log-space form), ``y_t = (h + r * c_prev_loc) * C_t + V_t``; when the token completes a block
    the carry snapshot becomes ``h`` and the local state is reset.

    Returns ``(y_t, new_state)``. By default ``state`` is left untouched and the new state owns new
    tensors (``c_prev_loc`` is shared with the old state except at a block boundary), as in the
    reference. With ``inplace=True`` the tensors of ``state`` are overwritten and ``state`` itself is
    returned with ``i`` advanced: no allocation besides ``y_t``.
    """
    _need_gpu(A_t, X_t, C_t, V_t, state.h_loc, state.c_prev_loc)
    log_mode = bool(state.use_log_r or use_log_a)
    X_t = X_t.contiguous()
    A_t = A_t.contiguous()
    C_t = C_t.to(X_t.dtype).contiguous()
    V_t = V_t.to(X_t.dtype).contiguous()
    y_t = torch.empty_like(X_t)
    boundary = state.i + 1 == state.block_len

    # the accumulator the kernel reads: a missing one starts at 1 (log: 0), as in the reference
    r_prev = state.log_r_pref if log_mode else state.r_pref
    if r_prev is None:
        r_prev = torch.zeros_like(A_t) if log_mode else torch.ones_like(A_t)
        fresh_r = True
    else:
        r_prev = r_prev.contiguous()
        fresh_r = False
    tiny = float(torch.finfo(A_t.dtype).tiny) if log_mode else 0.0

    if inplace:
        h_out, r_out = state.h_loc, r_prev
        c_out = state.c_prev_loc
    else:
        h_out = torch.empty_like(state.h_loc)
        r_out = r_prev if fresh_r else torch.empty_like(r_prev)
        c_out = torch.empty_like(state.c_prev_loc) if boundary else None
    _btp.jagged_step(
        A_t, X_t, C_t, V_t, y_t, state.h_loc, r_prev, state.c_prev_loc, h_out, r_out, c_out,
        boundary, use_log_a, log_mode, tiny,
    )
    i_next = 0 if boundary else state.i + 1
    c_new = c_out if boundary else state.c_prev_loc
    if inplace:
        state.i = i_next
        state.use_log_r = log_mode
        state.r_pref = None if log_mode else r_out
        state.log_r_pref = r_out if log_mode else None
        return y_t, state
    return y_t, JagState(
        h_loc=h_out,
        r_pref=None if log_mode else r_out,
        c_prev_loc=c_new,
        i=i_next,
        block_len=state.block_len,
        use_log_r=log_mode,
        log_r_pref=r_out if log_mode else None,
    )


@torch.no_grad()
def parallel_jagged(
    A: torch.Tensor,  # (B, H, L)      a if use_log_a=False, log(a) if True
    X: torch.Tensor,  # (B, H, D, L)   driving term per token (e.g., B*V)
    C: torch.Tensor,  # (B, H, D, L)
    V: torch.Tensor,  # (B, H, D, L)
    *,
    block_len: int,
    use_log_a: bool = False,
    state_dtype: torch.dtype | None = None,
) -> tuple[torch.Tensor, JagState]:
    """Prompt prefill (inference.py:281-360): ``Y = (block-local scans + one-hop carry) * C + V`` and
    the state after the last prompt token for :func:`step_jagged` to continue from. Any prompt length;
    no padding copies are made. The state tensors take ``V``'s dtype (``r_pref``: ``A``'s) unless
    ``state_dtype`` says otherwise (``torch.float32`` keeps them exact for 16-bit prompts)."""
    _need_gpu(A, X, C, V)
    Bsz, H, D, L = V.shape
    V = V.contiguous()
    X = X.to(V.dtype).contiguous()
    C = C.to(V.dtype).contiguous()
    A = A.contiguous()
    if A.dtype != V.dtype and A.dtype != torch.float32:
        A = A.float()
    Y = torch.empty_like(V)
    sdt = V.dtype if state_dtype is None else state_dtype
    h_tail = torch.empty((Bsz, H, D), device=V.device, dtype=sdt)
    c_prev_tail = torch.empty((Bsz, H, D), device=V.device, dtype=sdt)
    r_tail = torch.empty((Bsz, H), device=V.device, dtype=A.dtype if state_dtype is None else state_dtype)
    if L == 0:
        h_tail.zero_()
        c_prev_tail.zero_()
        r_tail.fill_(1.0)
    _btp.jagged_prefill(A, X, C, V, None, Y, h_tail, r_tail, c_prev_tail, block_len, use_log_a)
    state = JagState(
        h_loc=h_tail,
        r_pref=r_tail,
        c_prev_loc=c_prev_tail,
        i=L % block_len,
        block_len=block_len,
        use_log_r=False,
        log_r_pref=None,
    )
    return Y, state


# ---- decoding with the whole layer ------------------------------------------------------------------

@dataclass
class PhalanxStepState:
    """Streaming state of a ``Phalanx`` layer, fp32, updated in place by :func:`phalanx_step`:
    ``h_loc`` [B, H, 16] block-local state, ``r_pref`` [B, H] in-block gate product, ``c_prev_loc`` [B, H, 16]
    terminal local state of the last completed block, ``pos`` [B] int32 position of the next token inside
    its block (on the device: a captured step needs no host decision)."""

    h_loc: torch.Tensor
    r_pref: torch.Tensor
    c_prev_loc: torch.Tensor
    pos: torch.Tensor
    block_len: int = 16

    @classmethod
    def zeros(cls, batch: int, heads: int, device, block_len: int = 16) -> "PhalanxStepState":
        return cls(
            torch.zeros(batch, heads, 16, device=device),
            torch.ones(batch, heads, device=device),
            torch.zeros(batch, heads, 16, device=device),
            torch.zeros(batch, device=device, dtype=torch.int32),
            block_len,
        )


@torch.no_grad()
def phalanx_step(layer, x_t: torch.Tensor, state: PhalanxStepState, out: torch.Tensor | None = None) -> torch.Tensor:
    """One token through ``layer`` (a ``Phalanx``): ``x_t`` [B, dim] -> [B, dim]; ``state`` is updated in place.
    Equals position t of ``layer(x)`` for the sequence fed so far. Every op is stream-ordered and allocation
    apart, so the call can be recorded into a HIP graph (``torch.cuda.graph``) with fixed ``x_t`` / ``out``
    buffers and replayed once per token."""
    _need_gpu(x_t, state.h_loc)
    if layer.k != 2:  # a k = 1 layer has no carry between blocks; this step always applies the one-hop carry
        raise RuntimeError("phalanx_step needs a layer with k == 2")
    p = layer.param
    xc = x_t.to(p.compute_dtype)
    a, b, c, v = p.proj_a(xc), p.proj_b(xc), p.proj_c(xc), p.proj_v(xc)
    mixed = torch.empty_like(v)
    _btp.mix_step(a, b, c, v, mixed, state.h_loc, state.r_pref, state.c_prev_loc, state.pos, False,
                  state.block_len, layer.heads, layer.kv_heads)
    y = layer.proj_out(mixed)
    if out is not None:
        out.copy_(y)
        return out
    return y


@torch.no_grad()
def phalanx_prefill(layer, x: torch.Tensor) -> tuple[torch.Tensor, PhalanxStepState]:
    """A prompt ``x`` [B, L, dim] (any L >= 1) through ``layer``: returns the layer's output for it and the state
    after its last token, from which :func:`phalanx_step` continues. The whole blocks go through the fused
    forward kernel, which also leaves the hand-over state (``spear_phalanx_mix_prefill``: after a whole number of
    blocks the state is the last block's terminal local state, a zero block-local state and a gate product of
    one); the at most 15 tokens of a partial last block are projected together and stepped one kernel each."""
    _need_gpu(x)
    B, L, _ = x.shape
    p, bl = layer.param, 16
    if layer.k != 2:
        raise RuntimeError("phalanx_prefill needs a layer with k == 2")
    full = (L // bl) * bl
    state = PhalanxStepState.zeros(B, layer.heads, x.device, bl)
    xc = x.to(p.compute_dtype)
    parts = []
    if full > 0:
        a, b, c, v = (proj(xc[:, :full]) for proj in (p.proj_a, p.proj_b, p.proj_c, p.proj_v))
        mixed = torch.empty_like(v)
        _btp.mix_forward(a, b, c, v, mixed, layer.heads, layer.kv_heads, c_prev_tail=state.c_prev_loc)
        parts.append(mixed)
    if L > full:
        a, b, c, v = (proj(xc[:, full:]).transpose(0, 1).contiguous() for proj in (p.proj_a, p.proj_b, p.proj_c, p.proj_v))
        tail = torch.empty_like(v)  # [tokens, B, dim]
        for t in range(L - full):
            _btp.mix_step(a[t], b[t], c[t], v[t], tail[t], state.h_loc, state.r_pref, state.c_prev_loc, state.pos, False,
                          bl, layer.heads, layer.kv_heads)
        parts.append(tail.transpose(0, 1))
    return layer.proj_out(parts[0] if len(parts) == 1 else torch.cat(parts, dim=1)), state
