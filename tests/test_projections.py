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


@pytest.mark.gpu
@pytest.mark.parametrize("B,L,dim,heads,kv_heads", [(2, 64, 128, 8, 8), (3, 128, 256, 16, 4), (96, 128, 256, 16, 16), (72, 128, 192, 12, 3)])
def test_project_and_mix_matches_the_mixing_op_on_linear_autograd(B, L, dim, heads, kv_heads):
    """``project_and_mix`` (packed gradient buffer, bias gradients from the kernel's sums) against
    ``phalanx_mix`` applied to four ``nn.Linear`` outputs under plain autograd."""
    from spear_amd.ops.btp import phalanx_mix

    mods = _modules(dim, heads, kv_heads, torch.bfloat16, "cuda:0", 11)[:4]
    g = torch.Generator(device="cpu").manual_seed(12)
    x0 = torch.randn(B, L, dim, generator=g).bfloat16().to("cuda:0")
    dout = torch.randn(B, L, heads * 16, generator=g).bfloat16().to("cuda:0")

    def run(custom):
        for m in mods:
            m.zero_grad(set_to_none=True)
        x = x0.clone().requires_grad_(True)
        out = (pj.project_and_mix(x, *mods, heads, kv_heads) if custom
               else phalanx_mix(*(m(x) for m in mods), heads, kv_heads))
        out.backward(dout)
        return out.detach(), [x.grad] + [p.grad for m in mods for p in m.parameters()]

    (out, grads), (ref_out, ref_grads) = run(True), run(False)
    assert torch.equal(out, ref_out)
    names = ["x", "w_a", "b_a", "w_b", "b_b", "w_c", "b_c", "w_v"]
    for name, got, ref in zip(names, grads, ref_grads):
        assert got.shape == ref.shape, name
        got, ref = got.float(), ref.float()
        scale = ref.abs().max().item()
        # bf16 results of fp32-accumulated sums; the bias sums are taken before the gradients' rounding
        assert (got - ref).abs().max().item() <= 2 ** -6 * scale, (name, (got - ref).abs().max().item() / scale)
