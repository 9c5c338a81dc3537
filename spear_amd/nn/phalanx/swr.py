"""Phalanx: sliding-window-recurrence token mixer with sigmoid gates, head_dim fixed at 16.

Drop-in for the reference's ``spear.nn.phalanx.swr`` (spear/nn/phalanx/swr.py): the same three
classes with the same constructor arguments, attribute names, ``state_dict`` keys
(``param.proj_{a,b,c,v}.*``, ``proj_out.weight``) and parameter creation order (so a given seed
initialises identical weights).

    A = sigmoid(proj_a(x))            decay per head and step        [B, H, L]
    X = sigmoid(proj_b(x)) * proj_v(x)  gated input                   [B, H, 16, L]
    C = proj_c(x),  V = proj_v(x)                                      [B, H, 16, L]
    y = proj_out( (recurrence(A, X) * C + V)  laid out as [B, L, H*16] )

``method`` picks who evaluates the recurrence:
  ``"default"``           the HIP kernels through :func:`spear_amd.ops.btp.btp`
  ``"pytorch"``           the log-space PyTorch statement of the two-pass algorithm
  ``"pytorch_linspace"``  the linear-space PyTorch statement
  ``"fused"``             (addition) one HIP kernel for gates + recurrence + ``* C + V`` working
                          directly on the projection outputs, for any ``heads % kv_heads == 0``;
                          needs ``k == 2``
The choice is explicit; ``"default"`` and ``"fused"`` never degrade to a PyTorch path. Code written
against the reference says ``method="default"``; with ``SPEAR_PHALANX_DEFAULT=fused`` in the environment
such a layer runs the fused kernels wherever they apply (``k == 2``, 16-bit output) and
the stand-alone kernels elsewhere, without a change to the calling code.

On a GPU, from 8192 tokens per call on, the ``"default"`` and ``"fused"`` layers run their five
projections through :mod:`.projections` (same forward; weight gradients cut along the token axis, one
shared input gradient). The two ``"pytorch*"`` methods keep plain ``nn.Linear`` autograd, which is what the
other two are compared with.
"""

from __future__ import annotations

import os

import torch
import torch.nn as nn

from .projections import input_projections, linear, pays_off, project_and_mix

_HEAD_DIM = 16
_METHODS = ("default", "pytorch", "pytorch_linspace", "fused")


class KVRepeat(nn.Module):
    """Shares one key/value head among ``total_heads // kv_heads`` consecutive query heads
    (swr.py:21-126). With ``kv_heads == total_heads`` every method is a plain reshape."""

    def __init__(self, kv_heads: int, total_heads: int):
        super().__init__()
        if total_heads % kv_heads != 0:
            raise ValueError(f"total_heads ({total_heads}) must be divisible by kv_heads ({kv_heads})")
        self.kv_heads = kv_heads
        self.total_heads = total_heads
        self.kv_groups = total_heads // kv_heads
        self.enabled = kv_heads < total_heads
        if self.enabled:
            # query head h reads kv head h // kv_groups: [0,0,..,1,1,..]
            self.register_buffer("kv_indices", torch.arange(total_heads) // self.kv_groups, persistent=False)

    def _gather(self, t: torch.Tensor) -> torch.Tensor:
        return t.index_select(1, self.kv_indices)

    def forward(self, tensor: torch.Tensor, pattern: str = "b h d l") -> torch.Tensor:
        return self._gather(tensor) if self.enabled else tensor

    def reshape_for_kv(self, tensor: torch.Tensor, batch: int, head_dim: int, length: int) -> torch.Tensor:
        return tensor.view(batch, self.kv_heads, head_dim, length)

    def expand_and_reshape(self, tensor: torch.Tensor, batch: int, head_dim: int, length: int) -> torch.Tensor:
        per_kv_head = tensor.view(batch, self.kv_heads, head_dim, length)
        return self._gather(per_kv_head) if self.enabled else per_kv_head

    def expand_flat(self, tensor: torch.Tensor, head_dim: int) -> torch.Tensor:
        if not self.enabled:
            return tensor
        B, _, L = tensor.shape
        return self._gather(tensor.view(B, self.kv_heads, head_dim, L)).view(B, self.total_heads * head_dim, L)


class SigmoidA(nn.Module):
    """The four input projections and their gates (swr.py:129-221). Inputs are cast to bf16
    before the projections, so the layer is meant to be built with ``dtype=torch.bfloat16``."""

    def __init__(
        self,
        dim: int,
        heads: int,
        head_dim: int,
        dtype: torch.dtype = torch.bfloat16,
        mixed_precision: bool = True,
        kv_heads: int | None = None,
    ):
        super().__init__()
        self.heads = heads
        self.head_dim = head_dim
        self.dim = dim
        self.dtype = dtype
        self.compute_dtype = torch.bfloat16
        self.kv_heads = heads if kv_heads is None else kv_heads
        if heads % self.kv_heads != 0:
            raise ValueError(f"heads ({heads}) must be divisible by kv_heads ({self.kv_heads})")
        self.kv_repeat = KVRepeat(self.kv_heads, heads)
        self.dim_bvc = 3 * heads * head_dim
        self.dim_a = heads
        self.token_sliced_backward = False  # set by Phalanx for the methods that run HIP kernels

        # creation order fixes the RNG draw order of the default initialisation
        self.proj_a = nn.Linear(dim, heads, bias=True, dtype=dtype)
        self.proj_b = nn.Linear(dim, self.kv_heads * head_dim, bias=True, dtype=dtype)
        self.proj_c = nn.Linear(dim, self.kv_heads * head_dim, bias=True, dtype=dtype)
        self.proj_v = nn.Linear(dim, heads * head_dim, bias=False, dtype=dtype)

    def project(self, x: torch.Tensor):
        """``(proj_a(x), proj_b(x), proj_c(x), proj_v(x))`` as [B, L, features] tensors."""
        xc = x.to(self.compute_dtype)
        if self.token_sliced_backward and pays_off(xc):
            return input_projections(xc, self.proj_a, self.proj_b, self.proj_c, self.proj_v)
        return tuple(p(xc) for p in (self.proj_a, self.proj_b, self.proj_c, self.proj_v))

    def _compute_base_projections(self, x: torch.Tensor):
        """Raw projections as [B, features, L] views (time last, not yet contiguous)."""
        return tuple(t.transpose(1, 2) for t in self.project(x))

    def forward_fused_gates(self, x: torch.Tensor) -> torch.Tensor:
        """Packed ``[B_gate, V, C, A]`` along the feature axis: ``[B, 3*H*16 + H, L]``."""
        a_logits, b_kv, c_kv, v = self._compute_base_projections(x)
        return torch.cat(
            [self.kv_repeat.expand_flat(b_kv, self.head_dim), v, self.kv_repeat.expand_flat(c_kv, self.head_dim), a_logits],
            dim=1,
        )

    def forward_axcv(self, x: torch.Tensor):
        """``(A [B,H,L], X [B,H,16,L], C [B,H,16,L], V [B,H,16,L])`` for the recurrence."""
        B, L, _ = x.shape
        H, DH = self.heads, self.head_dim
        a_logits, b_kv, c_kv, v_flat = self._compute_base_projections(x)
        V = v_flat.view(B, H, DH, L)
        gate = torch.sigmoid(self.kv_repeat.expand_and_reshape(b_kv, B, DH, L))
        C = self.kv_repeat.expand_and_reshape(c_kv, B, DH, L)
        return torch.sigmoid(a_logits), gate * V, C, V


class Phalanx(nn.Module):
    def __init__(
        self,
        dim: int,
        heads: int | None = None,
        length: int = 2048,
        method: str = "default",
        dtype: torch.dtype = torch.float32,
        k: int = 2,
        wpb: int = 32,
        output_dtype: torch.dtype | None = None,
        block_size: int = 16,
        kv_heads: int | None = None,
    ):
        super().__init__()
        if heads is None:
            if dim % _HEAD_DIM != 0:
                raise ValueError(f"dim ({dim}) must be divisible by 16")
            heads = dim // _HEAD_DIM
        else:
            if dim % heads != 0:
                raise ValueError(f"dim ({dim}) must be divisible by heads ({heads})")
            if dim // heads != _HEAD_DIM:
                raise ValueError(f"head_dim must be 16, got {dim // heads}. Use heads=dim//16 or leave heads=None")
        if method not in _METHODS:
            raise ValueError(f"method must be one of 'default', 'pytorch', 'pytorch_linspace', got {method}")
        if method == "fused" and k != 2:
            raise ValueError("method 'fused' needs k == 2")

        self.dim = dim
        self.heads = heads
        self.head_dim = _HEAD_DIM
        self.length = -(-length // 16) * 16
        self.method = method
        self.dtype = dtype
        self.compute_dtype = torch.bfloat16
        self.k = k
        self.wpb = wpb
        self.output_dtype = dtype if output_dtype is None else output_dtype
        self.block_size = block_size
        self.kv_heads = heads if kv_heads is None else kv_heads

        self.param = SigmoidA(dim, heads, self.head_dim, dtype=dtype, kv_heads=kv_heads)
        self.proj_out = nn.Linear(dim, dim, bias=False, dtype=dtype)
        self.param.token_sliced_backward = method in ("default", "fused")

        runs_fused = method == "fused" or (
            method == "default" and os.environ.get("SPEAR_PHALANX_DEFAULT", "") == "fused"
            and k == 2 and self.output_dtype == self.compute_dtype
        )
        if method == "default" and not runs_fused:
            from spear_amd.ops.btp import btp

            self.btp_module = btp
            self._forward_fn = self._forward_default
        elif runs_fused:
            from spear_amd.ops.btp import phalanx_mix

            self.mix_module = phalanx_mix
            self._forward_fn = self._forward_fused
        else:
            from spear_amd.ops.btp import reference

            self.pytorch_block_two_pass = (
                reference.block_two_pass_log if method == "pytorch" else reference.block_two_pass_linspace
            )
            self._forward_fn = self._forward_pytorch

    def _mix_and_project(self, h: torch.Tensor, C: torch.Tensor, V: torch.Tensor) -> torch.Tensor:
        out = h * C + V  # [B, H, 16, L]
        B, H, DH, L = out.shape
        return self._project_out(out.permute(0, 3, 1, 2).reshape(B, L, H * DH))

    def _project_out(self, mixed: torch.Tensor) -> torch.Tensor:
        if self.param.token_sliced_backward and pays_off(mixed):
            return linear(mixed, self.proj_out)
        return self.proj_out(mixed)

    def _forward_pytorch(self, x: torch.Tensor) -> torch.Tensor:
        A, X, C, V = self.param.forward_axcv(x)
        return self._mix_and_project(self.pytorch_block_two_pass(A, X, self.block_size), C, V)

    def _forward_default(self, x: torch.Tensor) -> torch.Tensor:
        A, X, C, V = self.param.forward_axcv(x)
        return self._mix_and_project(self.btp_module(A, X, self.k, self.wpb, self.output_dtype), C, V)

    def _forward_fused(self, x: torch.Tensor) -> torch.Tensor:
        p = self.param
        xc = x.to(p.compute_dtype)
        if xc.dim() == 3 and pays_off(xc):
            mixed = project_and_mix(xc, p.proj_a, p.proj_b, p.proj_c, p.proj_v, self.heads, self.kv_heads)
        else:
            mixed = self.mix_module(*p.project(xc), self.heads, self.kv_heads)
        return self._project_out(mixed)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self._forward_fn(x)
