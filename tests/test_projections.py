"""The layer's projection functions (spear_amd/nn/phalanx/projections.py) against plain ``nn.Linear``
autograd: same forward, same gradients up to the rounding of an fp32 sum associated differently."""

import pytest
import torch
import torch.nn as nn

from spear_amd.nn.phalanx import projections as pj


def _modules(dim, heads, kv_heads, dtype, device, seed):
    torch.manual_seed(seed)
    mods = (nn.Linear(dim, heads, dtype=dtype), nn.Linear(dim, kv_heads * 16, dtype=dtype),
            nn.Linear(dim, kv_heads * 16, dtype=dtype), nn.Linear(dim, heads * 16, bias=False, dtype=dtype),
            nn.Linear(dim, dim, bias=False, dtype=dtype))
    return [m.to(device) for m in mods]


def _both_ways(B, L, dim, heads, kv_heads, dtype, device, seed=0):
    mods = _modules(dim, heads, kv_heads, dtype, device, seed)
    g = torch.Generator(device="cpu").manual_seed(seed + 1)
    x0 = torch.randn(B, L, dim, generator=g).to(dtype).to(device)
    weights = [torch.randn(B, L, m.out_features, generator=g).to(dtype).to(device) for m in mods]

    def run(custom):
        for m in mods:
            m.zero_grad(set_to_none=True)
        x = x0.clone().requires_grad_(True)
        if custom:
            outs = list(pj.input_projections(x, *mods[:4])) + [pj.linear(x, mods[4])]
        else:
            outs = [m(x) for m in mods]
        sum((o.float() * w.float()).sum() for o, w in zip(outs, weights)).backward()
        grads = [x.grad] + [p.grad for m in mods for p in m.parameters()]
        return [o.detach() for o in outs], grads

    return run(True), run(False)


def test_slice_count_cuts_only_long_token_axes_evenly():
    assert pj.slice_count(256, 512, 512) == 1
    assert pj.slice_count(131072, 512, 512) == 64
    assert pj.slice_count(131072, 1024, 1024) == 16
    assert pj.slice_count(131072, 32, 512) == 64
    for M in (131072, 3 * 4096, 5 * 2048, 7 * 1024 + 16, 1 << 20):
        for N, K in ((32, 512), (512, 512), (2048, 2048)):
            s = pj.slice_count(M, N, K)
            assert M % s == 0 and (s == 1 or M // s >= 1024) and s <= 64


def test_projection_functions_equal_linear_autograd_in_fp32_on_the_cpu():
    (outs, grads), (ref_outs, ref_grads) = _both_ways(2, 48, 64, 4, 2, torch.float32, "cpu")
    for o, r in zip(outs, ref_outs):
        assert torch.equal(o, r)
    for got, ref in zip(grads, ref_grads):
        torch.testing.assert_close(got, ref, rtol=1e-5, atol=1e-5)


def test_unused_outputs_and_frozen_parameters():
    mods = _modules(32, 2, 2, torch.float32, "cpu", 3)
    mods[1].weight.requires_grad_(False)
    x = torch.randn(3, 16, 32, requires_grad=True)
    a, b, c, v = pj.input_projections(x, *mods[:4])
    (a.sum() + 2 * v.sum()).backward()          # b and c unused
    x2 = x.detach().clone().requires_grad_(True)
    (mods[0](x2).sum() + 2 * mods[3](x2).sum()).backward()
    torch.testing.assert_close(x.grad, x2.grad)
    assert mods[1].weight.grad is None


@pytest.mark.gpu
@pytest.mark.parametrize("B,L,dim,heads,kv_heads", [(2, 128, 256, 16, 16), (96, 128, 256, 16, 4), (256, 128, 512, 32, 32)])
def test_token_sliced_gradients_match_linear_autograd_on_the_gpu(B, L, dim, heads, kv_heads):
    """The larger cases cut the token axis (slice_count > 1). bf16 results of the same fp32-accumulated
    products: equal up to one rounding of the result."""
    (outs, grads), (ref_outs, ref_grads) = _both_ways(B, L, dim, heads, kv_heads, torch.bfloat16, "cuda:0")
    if B * L >= 8192:
        assert pj.slice_count(B * L, dim, dim) > 1
    for o, r in zip(outs, ref_outs):
        assert torch.equal(o, r)
    for got, ref in zip(grads, ref_grads):
        got, ref = got.float(), ref.float()
        scale = ref.abs().max().item()
        assert (got - ref).abs().max().item() <= 2 ** -6 * scale, (got - ref).abs().max().item() / scale
