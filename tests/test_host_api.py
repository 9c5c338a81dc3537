"""Host-side behaviour that needs no GPU: the op's argument checks and messages (mirroring
csrc/btp/_bindings.cu:19-60 and spear/ops/btp/interface.py:137-139 of the reference), the
registered custom ops, the package surface, and the Phalanx layer's construction rules."""

import numpy as np
import pytest
import torch

import spear_amd
from spear_amd import _btp
from spear_amd.nn.phalanx import KVRepeat, Phalanx, SigmoidA
from spear_amd.ops.btp import interface


def _cpu_args(B=1, H=2, L=32, dtype=torch.bfloat16):
    coeff = torch.rand(B, H, L).to(dtype)
    x = torch.randn(B, H, 16, L).to(dtype)
    y = torch.empty(B, H, 16, L, dtype=torch.float32)
    ck = torch.empty(B, H, L // 16, 16, dtype=torch.float32)
    return coeff, x, y, ck


def test_package_surface():
    assert spear_amd.__version__ == "0.1.0"
    assert spear_amd.btp is interface.btp
    assert spear_amd.Phalanx is Phalanx and spear_amd.SigmoidA is SigmoidA
    assert (interface.DH, interface.BLK) == (16, 16)
    assert interface.SUPPORTED_WPB == [4, 8, 16, 32]
    assert (interface.WPB_K1_DEFAULT, interface.WPB_K2_DEFAULT) == (8, 32)


def test_custom_ops_are_registered_with_the_reference_schemas():
    fwd = torch.ops.spear_btp.forward.default._schema
    bwd = torch.ops.spear_btp.backward.default._schema
    assert [a.name for a in fwd.arguments] == ["coeff", "x", "y", "checkpoint", "k", "wpb"]
    assert [a.name for a in bwd.arguments] == ["coeff", "x", "dy", "checkpoint", "dx", "dA", "k", "wpb"]
    assert [a.name for a in fwd.arguments if a.alias_info and a.alias_info.is_write] == ["y", "checkpoint"]
    assert [a.name for a in bwd.arguments if a.alias_info and a.alias_info.is_write] == ["dx", "dA"]


def test_non_gpu_tensors_are_rejected_like_the_reference():
    coeff, x, y, ck = _cpu_args()
    with pytest.raises(RuntimeError, match="All tensors must be CUDA"):
        _btp.forward(coeff, x, y, ck, 2, 32)
    with pytest.raises(RuntimeError, match="coeff, x, dy, checkpoint must be CUDA"):
        _btp.backward(coeff, x, y, ck, torch.empty_like(x), torch.empty(1, 2, 32), 2, 32)


def test_there_is_no_cpu_fallback_for_the_op():
    coeff, x, _, _ = _cpu_args()
    with pytest.raises((RuntimeError, NotImplementedError)):
        interface.btp(coeff, x)


def test_missing_library_is_a_loud_error(monkeypatch, tmp_path):
    monkeypatch.setattr(_btp, "_lib", None)
    monkeypatch.setenv("SPEAR_BTP_LIBRARY", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="could not be loaded"):
        _btp.load_library()


@pytest.mark.parametrize(
    "mutate,msg",
    [
        (lambda a: a.__setitem__("x", a["x"][0]), r"x must be \[B, H, 16, L\]"),
        (lambda a: a.__setitem__("x", torch.empty(1, 2, 8, 32, dtype=torch.bfloat16)), "Channel dim"),
        (lambda a: a.__setitem__("k", 3), "k must be 1 or 2"),
        (lambda a: a.__setitem__("wpb", 5), "Unsupported WPB value: 5"),
        (lambda a: a.__setitem__("coeff", a["coeff"].float()), "coeff must be float16 or bfloat16"),
        (lambda a: a.__setitem__("x", a["x"].half()), "x dtype must match coeff"),
        (lambda a: a.__setitem__("y", a["y"].half()), "y must be float32 or match x dtype"),
        (lambda a: a.__setitem__("ck", a["ck"].half()), "checkpoint must be float32"),
    ],
)
def test_forward_checks_fire_in_the_reference_order(monkeypatch, mutate, msg):
    # pretend the tensors live on the GPU so that the later checks are reached
    monkeypatch.setattr(torch.Tensor, "is_cuda", property(lambda self: True))
    coeff, x, y, ck = _cpu_args()
    a = dict(coeff=coeff, x=x, y=y, ck=ck, k=2, wpb=32)
    mutate(a)
    with pytest.raises(RuntimeError, match=msg):
        _btp.forward(a["coeff"], a["x"], a["y"], a["ck"], a["k"], a["wpb"])


def test_shape_mismatches_raise_instead_of_reading_out_of_bounds(monkeypatch):
    monkeypatch.setattr(torch.Tensor, "is_cuda", property(lambda self: True))
    coeff, x, y, ck = _cpu_args()
    with pytest.raises(RuntimeError, match="coeff must have shape"):
        _btp.forward(coeff[:, :1], x, y, ck, 2, 32)
    with pytest.raises(RuntimeError, match="x must be contiguous"):
        strided = torch.randn(1, 2, 16, 64).bfloat16()[..., ::2]
        _btp.forward(coeff, strided, y, ck, 2, 32)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        c2 = torch.rand(1, 2, 24).bfloat16()
        x2 = torch.randn(1, 2, 16, 24).bfloat16()
        _btp.forward(c2, x2, torch.empty(1, 2, 16, 24), torch.empty(1, 2, 1, 16), 2, 32)


def test_python_level_asserts():
    coeff = torch.rand(1, 2, 24).bfloat16()
    with pytest.raises(AssertionError, match="multiple of 16"):
        interface.btp(coeff, torch.randn(1, 2, 16, 24).bfloat16())
    with pytest.raises(AssertionError, match="Channel dimension"):
        interface.btp(torch.rand(1, 2, 32).bfloat16(), torch.randn(1, 2, 8, 32).bfloat16())
    with pytest.raises(AssertionError, match="WPB"):
        interface.btp(torch.rand(1, 2, 32).bfloat16(), torch.randn(1, 2, 16, 32).bfloat16(), wpb=7)


# ---- Phalanx layer ------------------------------------------------------------------------------

def test_phalanx_validation_errors():
    with pytest.raises(ValueError, match="divisible by 16"):
        Phalanx(dim=100)
    with pytest.raises(ValueError, match="head_dim must be 16"):
        Phalanx(dim=256, heads=8)
    with pytest.raises(ValueError, match="divisible by heads"):
        Phalanx(dim=256, heads=7)
    with pytest.raises(ValueError, match="method must be one of"):
        Phalanx(dim=256, method="cuda")
    with pytest.raises(ValueError, match="divisible by kv_heads"):
        Phalanx(dim=256, kv_heads=5)
    with pytest.raises(ValueError):
        KVRepeat(3, 16)


def test_phalanx_attributes_and_state_dict_keys():
    layer = Phalanx(dim=256, length=100, method="default", dtype=torch.bfloat16)  # needs no GPU to build
    assert (layer.heads, layer.head_dim, layer.length, layer.k, layer.wpb) == (16, 16, 112, 2, 32)
    assert layer.output_dtype == torch.bfloat16 and layer.kv_heads == 16
    assert set(layer.state_dict()) == {
        "param.proj_a.weight", "param.proj_a.bias", "param.proj_b.weight", "param.proj_b.bias",
        "param.proj_c.weight", "param.proj_c.bias", "param.proj_v.weight", "proj_out.weight",
    }
    assert layer.param.proj_a.weight.shape == (16, 256)
    assert layer.param.proj_v.weight.shape == (256, 256) and layer.param.proj_v.bias is None


def test_phalanx_default_init_is_reproducible_across_methods():
    torch.manual_seed(7)
    a = Phalanx(dim=128, method="pytorch", dtype=torch.bfloat16)
    torch.manual_seed(7)
    b = Phalanx(dim=128, method="default", dtype=torch.bfloat16)
    for (ka, va), (kb, vb) in zip(a.state_dict().items(), b.state_dict().items()):
        assert ka == kb and torch.equal(va, vb)


@pytest.mark.parametrize("method", ["pytorch", "pytorch_linspace"])
@pytest.mark.parametrize("kv_heads", [None, 2])
def test_phalanx_pytorch_methods_run_on_cpu(method, kv_heads):
    torch.manual_seed(0)
    layer = Phalanx(dim=128, length=64, method=method, dtype=torch.bfloat16, kv_heads=kv_heads)
    x = torch.randn(2, 64, 128).bfloat16()
    y = layer(x)
    assert y.shape == (2, 64, 128) and y.dtype == torch.bfloat16 and torch.isfinite(y.float()).all()
    y.float().sum().backward()
    assert all(p.grad is not None for p in layer.parameters())
    if kv_heads:
        assert layer.param.proj_b.weight.shape == (kv_heads * 16, 128)
        assert not any("kv_indices" in k for k in layer.state_dict())


def test_log_and_linear_space_layers_agree():
    torch.manual_seed(1)
    a = Phalanx(dim=128, length=64, method="pytorch", dtype=torch.bfloat16)
    b = Phalanx(dim=128, length=64, method="pytorch_linspace", dtype=torch.bfloat16)
    b.load_state_dict(a.state_dict())
    x = torch.randn(2, 64, 128).bfloat16()
    assert (a(x).float() - b(x).float()).abs().max() <= 1e-1  # layer forward limit of the reference tests


def test_fused_gates_packing_order():
    torch.manual_seed(2)
    p = SigmoidA(64, 4, 16, dtype=torch.bfloat16, kv_heads=2)
    x = torch.randn(1, 32, 64).bfloat16()
    packed = p.forward_fused_gates(x)
    assert packed.shape == (1, 3 * 4 * 16 + 4, 32)
    a_logits, b_kv, c_kv, v = p._compute_base_projections(x)
    assert torch.equal(packed[:, 64:128], v) and torch.equal(packed[:, -4:], a_logits)
    assert torch.equal(packed[:, :16], b_kv[:, :16]) and torch.equal(packed[:, 16:32], b_kv[:, :16])  # heads 0,1 share kv head 0


# ---- entry points added next to the reference API ------------------------------------------------

def test_added_ops_are_registered():
    names = {"forward_log": ["gate", "x", "y", "k"], "backward_log": ["gate", "x", "dy", "dx", "dgate", "k"],
             "mix_forward": ["a_logits", "b_logits", "c", "v", "out", "heads", "kv_heads"],
             "mix_backward": ["a_logits", "b_logits", "c", "v", "dout", "da", "db", "dc", "dv", "heads", "kv_heads"]}
    for op, args in names.items():
        schema = getattr(torch.ops.spear_btp, op).default._schema
        assert [a.name for a in schema.arguments] == args


def test_log_gate_host_checks(monkeypatch):
    from spear_amd import btp_log

    gate = -torch.rand(1, 2, 32)
    x = torch.randn(1, 2, 16, 32).bfloat16()
    with pytest.raises(RuntimeError, match="All tensors must be CUDA"):
        _btp.forward_log(gate, x, torch.empty(1, 2, 16, 32), 2)
    with pytest.raises((RuntimeError, NotImplementedError)):
        btp_log(gate, x)  # no CPU fallback
    monkeypatch.setattr(torch.Tensor, "is_cuda", property(lambda self: True))
    with pytest.raises(RuntimeError, match="gate must be float32"):
        _btp.forward_log(gate.bfloat16(), x, torch.empty(1, 2, 16, 32), 2)
    with pytest.raises(RuntimeError, match="x must be float16 or bfloat16"):
        _btp.forward_log(gate, x.float(), torch.empty(1, 2, 16, 32), 2)
    with pytest.raises(RuntimeError, match="gate must have shape"):
        _btp.forward_log(gate[:, :1], x, torch.empty(1, 2, 16, 32), 2)
    with pytest.raises(RuntimeError, match="dgate must be float32"):
        _btp.backward_log(gate, x, x, torch.empty_like(x), torch.empty(1, 2, 32).bfloat16(), 2)


def test_fused_mix_host_checks(monkeypatch):
    a, b, c, v = torch.randn(1, 32, 4).bfloat16(), torch.randn(1, 32, 64).bfloat16(), torch.randn(1, 32, 64).bfloat16(), torch.randn(1, 32, 64).bfloat16()
    out = torch.empty_like(v)
    with pytest.raises(RuntimeError, match="All tensors must be CUDA"):
        _btp.mix_forward(a, b, c, v, out, 4, 4)
    monkeypatch.setattr(torch.Tensor, "is_cuda", property(lambda self: True))
    with pytest.raises(RuntimeError, match="divisible by kv_heads"):
        _btp.mix_forward(a, b, c, v, out, 4, 3)
    with pytest.raises(RuntimeError, match="b_logit must have shape"):
        _btp.mix_forward(a, b, c, v, out, 4, 2)
    with pytest.raises(RuntimeError, match="share one dtype"):
        _btp.mix_forward(a, b.half(), c, v, out, 4, 4)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        _btp.mix_forward(a[:, :24].contiguous(), b[:, :24].contiguous(), c[:, :24].contiguous(), v[:, :24].contiguous(), out[:, :24].contiguous(), 4, 4)


def test_fused_method_construction_rules():
    assert Phalanx(dim=32, method="fused", dtype=torch.bfloat16).heads == 2   # any head count
    assert Phalanx(dim=96, method="fused", dtype=torch.bfloat16, kv_heads=2).param.kv_repeat.kv_groups == 3
    with pytest.raises(ValueError, match="k == 2"):
        Phalanx(dim=128, method="fused", k=1, dtype=torch.bfloat16)
    layer = Phalanx(dim=128, method="fused", dtype=torch.bfloat16, kv_heads=2)  # builds without a GPU
    assert layer.kv_heads == 2 and layer.heads == 8


def test_oracle_fused_composition_matches_torch_composition():
    """The float64 composition used to check the fused kernel, against the same function written
    with torch ops and the float64 reference recurrence."""
    import numpy as np

    from oracle import btp_oracle as orc
    from spear_amd.ops.btp.reference import block_two_pass_ref

    B, L, H, Hkv = 2, 48, 8, 2
    g = torch.Generator().manual_seed(9)
    a, b, c, v = (torch.randn(B, L, n, generator=g, dtype=torch.float64) for n in (H, Hkv * 16, Hkv * 16, H * 16))
    heads = lambda t, h: t.view(B, L, h, 16).permute(0, 2, 3, 1)
    A = torch.sigmoid(a).transpose(1, 2).contiguous()
    G = torch.sigmoid(heads(b, Hkv)).repeat_interleave(H // Hkv, 1)
    C = heads(c, Hkv).repeat_interleave(H // Hkv, 1)
    V = heads(v, H)
    want = (block_two_pass_ref(A, (G * V).contiguous()) * C + V).permute(0, 3, 1, 2).reshape(B, L, H * 16)
    got = orc.phalanx_mix_forward(a.numpy(), b.numpy(), c.numpy(), v.numpy(), H, Hkv)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-11, atol=1e-12)


def test_oracle_fused_backward_matches_torch_autograd():
    import numpy as np

    from oracle import btp_oracle as orc
    from spear_amd.ops.btp.reference import block_two_pass_ref

    B, L, H, Hkv = 2, 48, 8, 2
    g = torch.Generator().manual_seed(9)
    a, b, c, v = (torch.randn(B, L, n, generator=g, dtype=torch.float64, requires_grad=True) for n in (H, Hkv * 16, Hkv * 16, H * 16))
    dout = torch.randn(B, L, H * 16, generator=g, dtype=torch.float64)
    heads = lambda t, h: t.view(B, L, h, 16).permute(0, 2, 3, 1)
    A = torch.sigmoid(a).transpose(1, 2).contiguous()
    G = torch.sigmoid(heads(b, Hkv)).repeat_interleave(H // Hkv, 1)
    C = heads(c, Hkv).repeat_interleave(H // Hkv, 1)
    out = (block_two_pass_ref(A, (G * heads(v, H)).contiguous()) * C + heads(v, H)).permute(0, 3, 1, 2).reshape(B, L, H * 16)
    out.backward(dout)
    got = orc.phalanx_mix_backward(*(t.detach().numpy() for t in (a, b, c, v)), dout.numpy(), H, Hkv)
    for name, gg, t in zip("abcv", got, (a, b, c, v)):
        np.testing.assert_allclose(gg, t.grad.numpy(), rtol=1e-10, atol=1e-12, err_msg=f"d{name}")


def test_oracle_qkv_gate_form_matches_torch_composition_and_autograd():
    """out = q * btp(exp(gate), k * v) + v and its gradients (dgate w.r.t. the LOG decay), against the
    same expression in torch ops on the float64 reference recurrence, differentiated by autograd."""
    import numpy as np

    from oracle import btp_oracle as orc
    from spear_amd.ops.btp.reference import block_two_pass_ref

    B, L, H, Hkv = 2, 48, 8, 4
    g = torch.Generator().manual_seed(10)
    q, k = (torch.randn(B, L, Hkv * 16, generator=g, dtype=torch.float64, requires_grad=True) for _ in range(2))
    v = torch.randn(B, L, H * 16, generator=g, dtype=torch.float64, requires_grad=True)
    gate = (-torch.nn.functional.softplus(torch.randn(B, L, H, generator=g, dtype=torch.float64))).requires_grad_(True)
    dout = torch.randn(B, L, H * 16, generator=g, dtype=torch.float64)
    heads = lambda t, h: t.view(B, L, h, 16).permute(0, 2, 3, 1)
    A = torch.exp(gate).transpose(1, 2).contiguous()
    K = heads(k, Hkv).repeat_interleave(H // Hkv, 1)
    Q = heads(q, Hkv).repeat_interleave(H // Hkv, 1)
    out = (block_two_pass_ref(A, (K * heads(v, H)).contiguous()) * Q + heads(v, H)).permute(0, 3, 1, 2).reshape(B, L, H * 16)
    out.backward(dout)
    args = [t.detach().numpy() for t in (q, k, v, gate)]
    np.testing.assert_allclose(orc.qkv_gate_forward(*args, H, Hkv), out.detach().numpy(), rtol=1e-11, atol=1e-12)
    dgate, dk, dq, dv = orc.qkv_gate_backward(*args, dout.numpy(), H, Hkv)
    for name, got, t in (("dgate", dgate, gate), ("dk", dk, k), ("dq", dq, q), ("dv", dv, v)):
        np.testing.assert_allclose(got, t.grad.numpy(), rtol=1e-10, atol=1e-12, err_msg=name)


def test_default_method_can_be_sent_to_the_fused_kernels_by_environment(monkeypatch):
    from spear_amd import Phalanx

    plain = Phalanx(dim=64, dtype=torch.bfloat16)
    assert plain._forward_fn == plain._forward_default
    monkeypatch.setenv("SPEAR_PHALANX_DEFAULT", "fused")
    sent = Phalanx(dim=64, dtype=torch.bfloat16)
    assert sent.method == "default" and sent._forward_fn == sent._forward_fused
    assert list(sent.state_dict()) == list(plain.state_dict())
    # where the fused kernels do not apply the stand-alone kernels stay: k = 1, fp32 output; any head count is served
    for kwargs in (dict(dim=64, k=1), dict(dim=64, output_dtype=torch.float32)):
        layer = Phalanx(dtype=torch.bfloat16, **kwargs)
        assert layer._forward_fn == layer._forward_default
    layer = Phalanx(dim=32, dtype=torch.bfloat16)
    assert layer._forward_fn == layer._forward_fused
    # the explicit PyTorch methods are never rerouted
    layer = Phalanx(dim=64, dtype=torch.bfloat16, method="pytorch")
    assert layer._forward_fn == layer._forward_pytorch


def test_the_kernel_path_switch_is_read_from_the_environment():
    """SPEAR_BTP_PATH=mfma (read once, when the op module is imported) puts the matrix-core flag on both custom ops;
    anything else leaves the default recurrence kernels."""
    import os
    import subprocess
    import sys

    probe = ("from spear_amd.ops.btp import interface as i; from spear_amd import _btp; "
             "print(int(i._PATH_MFMA), int(bool(i._FORWARD_FLAGS & _btp.FLAG_PATH_MFMA)))")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for value, want in (("mfma", "1 1"), ("", "0 0"), ("scan", "0 0")):
        env = dict(os.environ, SPEAR_BTP_PATH=value, PYTHONPATH=root)
        out = subprocess.run([sys.executable, "-c", probe], env=env, capture_output=True, text=True, cwd=root, timeout=300)
        assert out.returncode == 0, out.stderr
        assert out.stdout.strip().splitlines()[-1] == want, (value, out.stdout)


def test_the_compiled_autograd_node_is_for_plain_eager_tensors_only():
    """btp() hands a call to the node compiled into the binding only when nothing has to see the custom ops:
    tensor subclasses, dispatch / function modes and functorch transforms get the Python node."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.utils._python_dispatch import TorchDispatchMode

    from spear_amd.ops.btp.interface import _plain_eager

    t = torch.ones(2, 2)
    assert _plain_eager(t, t)
    assert _plain_eager(t, torch.nn.Parameter(t))
    with FakeTensorMode() as mode:
        assert not _plain_eager(t, t)
        assert not _plain_eager(mode.from_tensor(t))
    assert not _plain_eager(mode.from_tensor(t))

    class Passthrough(TorchDispatchMode):
        def __torch_dispatch__(self, func, types, args=(), kwargs=None):
            return func(*args, **(kwargs or {}))

    with Passthrough():
        assert not _plain_eager(t)
    with torch.device("cpu"):  # a function mode
        assert not _plain_eager(t)
    seen = []
    torch.func.vmap(lambda row: seen.append(_plain_eager(row)) or row)(t)
    assert seen == [False]
    assert _plain_eager(t)


def test_streaming_module_surface_and_state_dataclass():
    from spear_amd.nn.phalanx import inference as inf

    # the reference's five names first, then the additions for decoding with the whole layer
    assert inf.__all__[:5] == ["jagged_band_infer_sequential", "JaggedBandState", "JagState", "step_jagged", "parallel_jagged"]
    assert inf.__all__[5:] == ["PhalanxStepState", "phalanx_prefill", "phalanx_step"]
    st = inf.JagState(torch.zeros(1, 2, 3), torch.ones(1, 2), torch.zeros(1, 2, 3), 5, 16)
    assert (st.use_log_r, st.log_r_pref) == (False, None)
    cl = st.clone_detached()
    cl.h_loc += 1
    assert float(st.h_loc.abs().max()) == 0.0 and cl.i == 5 and cl.block_len == 16
    # no CPU path: host tensors are refused before anything is computed
    with pytest.raises(RuntimeError, match="must be on a GPU"):
        inf.step_jagged(torch.ones(1, 2), torch.zeros(1, 2, 3), torch.ones(1, 2, 3), torch.zeros(1, 2, 3), st)
    with pytest.raises(RuntimeError, match="must be on a GPU"):
        inf.parallel_jagged(torch.ones(1, 2, 8), *(torch.zeros(1, 2, 3, 8) for _ in range(3)), block_len=4)
    with pytest.raises(AssertionError):
        inf.jagged_band_infer_sequential(torch.zeros(1, 2, 3, 8), torch.ones(1, 2, 7), 4)


def test_config1_cpu_path_reproduces_the_reference_layer():
    """Default initialisation draws the same weights in the same order as the reference's layer, and the
    bfloat16 CPU path gives the reference's output (bit-identical on the machine that wrote the vectors;
    one unit in the last place is allowed for another CPU's matmul kernels)."""
    from helpers import config1_layer_and_input, layer_reference_vectors

    v = layer_reference_vectors()
    layer, x = config1_layer_and_input("pytorch")
    assert np.array_equal(v["x.sums"], [x.double().sum().item(), x.double().square().sum().item()])
    for name, p in layer.state_dict().items():
        d, want = p.double(), v[f"param.{name}"]
        got = np.concatenate([[float(n) for n in p.shape] + [0.0] * (2 - p.dim()),
                              [d.sum().item(), d.square().sum().item()], d.flatten()[:8].numpy()])
        assert np.array_equal(got, want), f"{name}: default initialisation differs from the reference's"
    with torch.no_grad():
        y = layer(x)
    assert y.dtype == torch.bfloat16 and bool(v["y.dtype_is_bf16"][0])
    np.testing.assert_allclose(y[:, ::8, :].float().numpy(), v["y.every8"], rtol=2.0 ** -7, atol=2.0 ** -8)


def test_bench_reads_the_roofline_traffic_from_the_committed_profiles(tmp_path, monkeypatch):
    """`roofline.traffic` of the bench line is the "total MB" of the dominant kernel's row in the committed rocprofv3
    summary, with its source named; a missing file or row gives null, never a stale constant."""
    import os

    import bench

    got, src = bench.profiled_traffic("c3", "bwd_scan")
    assert src == {"file": "profiles/btp_kernels_c3_B1024_H32_L128.txt", "table": "HBM traffic per dispatch",
                   "row": "bwd_scan", "column": "total MB"}
    # within a few per cent of the algorithmic bytes of that launch (102 B x 4,194,304 units), and from the file
    assert 0.99 <= got / (102 * 1024 * 32 * 128) <= 1.05
    text = open(os.path.join(bench.ROOT, src["file"])).read()
    assert ("%.1f" % (got / 1e6)) in text
    for cfg in ("c4", "c5"):
        assert bench.profiled_traffic(cfg, "bwd_scan")[0] is not None
    assert bench.profiled_traffic("c3", "no_such_kernel") == (None, None)
    assert bench.profiled_traffic("c9", "bwd_scan") == (None, None)
    # a kernel whose name has a blank in it, and a file that lacks the table
    assert bench.profiled_traffic("c3", "fwd_scan log-gate")[0] is not None
    monkeypatch.setattr(bench, "PROFILES", str(tmp_path))
    (tmp_path / "btp_kernels_c3_x.txt").write_text("== kernel durations ==\nbwd_scan   1  2  3  4  5.0  1.0\n")
    assert bench.profiled_traffic("c3", "bwd_scan") == (None, None)
