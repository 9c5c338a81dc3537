"""Numerics runners for the Phalanx layer (counterpart of spear/nn/phalanx/runners.py:33-224):
seeded inputs, layer sets with identical weights, output and gradient comparisons."""

from __future__ import annotations

import torch

from spear_amd.testing.numerics import (
    DEFAULT_INPUT_DISTRIBUTION,
    InputDistributionConfig,
    compute_error_metrics,
    extract_layer_gradients,
    make_generator,
    manual_seed,
    maybe_synchronize,
    sample_tensor_from_spec,
)

from .swr import Phalanx

__all__ = [
    "sample_layer_inputs",
    "create_phalanx_layers",
    "run_layer_forward",
    "compare_layer_outputs",
    "compare_layer_gradients",
]


def _pick_device(device) -> torch.device:
    return torch.device(device or ("cuda" if torch.cuda.is_available() else "cpu"))


def sample_layer_inputs(
    B: int, L: int, dim: int, *, dtype: torch.dtype = torch.bfloat16, device: torch.device | None = None,
    seed: int | None = None, stress_scale: float = 1.0, distribution: InputDistributionConfig | None = None,
) -> torch.Tensor:
    """``[B, L, dim]`` activations, drawn on a CPU generator and moved to ``device``."""
    device = _pick_device(device)
    if seed is not None:
        manual_seed(seed, device)
    cpu = torch.device("cpu")
    dist = distribution or DEFAULT_INPUT_DISTRIBUTION
    x = sample_tensor_from_spec(
        dist.activation, (B, L, dim), dtype=dtype, generator=make_generator(cpu, seed), device=cpu,
        scale_multiplier=stress_scale,
    )
    return x.to(device)


def create_phalanx_layers(
    dim: int, length: int, *, methods: tuple[str, ...] = ("default", "pytorch", "pytorch_linspace"),
    dtype: torch.dtype = torch.bfloat16, k: int = 2, wpb: int = 32, output_dtype: torch.dtype | None = None,
    block_size: int = 16, kv_heads: int | None = None, device: torch.device | None = None, seed: int | None = None,
) -> dict[str, Phalanx]:
    """One layer per method; every layer after the first receives the first one's weights."""
    device = _pick_device(device)
    if seed is not None:
        manual_seed(seed, device)
    shared = dict(dim=dim, length=length, dtype=dtype, k=k, wpb=wpb, output_dtype=output_dtype,
                  block_size=block_size, kv_heads=kv_heads)
    layers = {method: Phalanx(method=method, **shared).to(device) for method in methods}
    weights = None
    for layer in layers.values():
        if weights is None:
            weights = layer.state_dict()
        else:
            layer.load_state_dict(weights)
    return layers


def run_layer_forward(layer: Phalanx, x: torch.Tensor, *, compile: bool = False, compile_opts: dict | None = None):
    fn = torch.compile(layer, **(compile_opts or {})) if compile else layer
    return fn(x)


def _check_reference(layers, reference_method):
    if reference_method not in layers:
        raise ValueError(f"Reference method '{reference_method}' not in layers")


def compare_layer_outputs(
    layers: dict[str, Phalanx],
    x: torch.Tensor,
    *,
    reference_method: str = "pytorch",
    compile: bool = False,
    compile_opts: dict | None = None,
) -> dict[str, dict[str, float]]:
    _check_reference(layers, reference_method)
    outs = {m: run_layer_forward(l, x, compile=compile, compile_opts=compile_opts) for m, l in layers.items()}
    maybe_synchronize(x.device)
    ref = outs[reference_method]
    return {m: compute_error_metrics(o, ref) for m, o in outs.items() if m != reference_method}


def compare_layer_gradients(
    layers: dict[str, Phalanx],
    x: torch.Tensor,
    *,
    grad_out: torch.Tensor | None = None,
    reference_method: str = "pytorch",
    compile: bool = False,
    compile_opts: dict | None = None,
) -> dict[str, dict[str, dict[str, float]]]:
    """Gradients w.r.t. the input and every parameter, each method against the reference method."""
    _check_reference(layers, reference_method)
    if grad_out is None:
        gen = torch.Generator().manual_seed(0)
        grad_out = torch.randn(x.shape, generator=gen, dtype=torch.float32).to(x.device)

    def gradients_of(layer: Phalanx) -> dict[str, torch.Tensor]:
        layer.zero_grad(set_to_none=True)
        xin = x.detach().clone().requires_grad_(True)
        run_layer_forward(layer, xin, compile=compile, compile_opts=compile_opts).backward(grad_out)
        wrt_input = torch.zeros_like(xin) if xin.grad is None else xin.grad.detach().clone()
        return {"x": wrt_input, **extract_layer_gradients(layer)}

    grads = {method: gradients_of(layer) for method, layer in layers.items()}
    maybe_synchronize(x.device)

    ref = grads[reference_method]
    return {
        m: {n: compute_error_metrics(t, ref[n]) for n, t in g.items() if n in ref}
        for m, g in grads.items()
        if m != reference_method
    }
