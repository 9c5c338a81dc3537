"""The drop-in surface beyond the C ABI: the reference's import name (`spear`), the compiled torch binding
that stands where the reference has `spear._btp` (csrc/btp/_bindings.cu:240-243), and the CMake target,
which must produce the same library as the hipcc recipe (same exported symbols, same ABI version)."""

import ctypes
import os
import shutil
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_the_reference_import_name_resolves_to_the_same_modules():
    import spear
    import spear_amd
    from spear import Phalanx, SigmoidA, btp  # spear/__init__.py:6-9 of the reference
    from spear.nn.phalanx import Phalanx as P2
    from spear.nn.phalanx.inference import JagState, parallel_jagged, step_jagged  # noqa: F401
    from spear.nn.phalanx.swr import KVRepeat  # noqa: F401
    from spear.ops.btp import btp as btp2
    from spear.ops.btp.interface import BLK, DH, SUPPORTED_WPB, WPB_K1_DEFAULT, WPB_K2_DEFAULT, _BTPFunction  # noqa: F401
    from spear.ops.btp.reference import block_two_pass_log, block_two_pass_ref  # noqa: F401
    from spear.ops.btp.runners import sample_inputs  # noqa: F401
    from spear.testing.numerics import metrics  # noqa: F401

    assert spear.__version__ == spear_amd.__version__ == "0.1.0"
    assert Phalanx is spear_amd.Phalanx is P2 and SigmoidA is spear_amd.SigmoidA
    assert btp is spear_amd.btp is btp2
    assert (DH, BLK, SUPPORTED_WPB, WPB_K1_DEFAULT, WPB_K2_DEFAULT) == (16, 16, [4, 8, 16, 32], 8, 32)
    import spear.ops.btp.interface as by_alias
    import spear_amd.ops.btp.interface as by_name

    assert by_alias is by_name and by_name.__name__ == "spear_amd.ops.btp.interface"
    assert by_name.__spec__.name == "spear_amd.ops.btp.interface"  # the alias leaves the module's own spec alone
    with pytest.raises(ImportError):
        import spear.no_such_module  # noqa: F401


def test_the_compiled_binding_is_what_spear_btp_names():
    from spear_amd import _btp

    import spear._btp as ext

    assert ext is _btp.load_extension()
    assert ext.abi_version() == _btp._ABI_VERSION == _btp.load_library().spear_btp_abi_version()
    for name in ("forward", "backward", "btp_autograd", "forward_log", "backward_log", "mix_forward", "mix_backward"):
        assert callable(getattr(ext, name))
    # the reference's positional signatures (csrc/btp/_bindings.cu:76-77, 152-153)
    assert ext.forward.__doc__.startswith("forward(coeff: torch.Tensor, x: torch.Tensor, y: torch.Tensor, checkpoint: torch.Tensor, k:")
    assert ext.backward.__doc__.startswith(
        "backward(coeff: torch.Tensor, x: torch.Tensor, dy: torch.Tensor, checkpoint: torch.Tensor, dx: torch.Tensor, dA: torch.Tensor, k:")
    # no GPU is needed to be refused: host tensors raise like TORCH_CHECK does in the reference (_bindings.cu:22)
    c = torch.ones(1, 1, 16, dtype=torch.bfloat16)
    x = torch.ones(1, 1, 16, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="All tensors must be CUDA"):
        ext.forward(c, x, torch.empty_like(x), torch.empty(1, 1, 1, 16), 2, 32)
    with pytest.raises(RuntimeError, match="must be CUDA"):
        ext.backward(c, x, x, torch.empty(1, 1, 1, 16), torch.empty_like(x), torch.empty(1, 1, 16), 2, 32)


def test_ops_are_registered_once_under_both_import_names():
    import spear.ops.btp  # noqa: F401
    import spear_amd.ops.btp  # noqa: F401

    for op in ("forward", "backward", "forward_log", "backward_log", "mix_forward", "mix_backward", "qkv_forward", "qkv_backward"):
        assert hasattr(torch.ops.spear_btp, op)
    schema = str(torch.ops.spear_btp.forward.default._schema)
    assert "Tensor(a2!) y" in schema and "Tensor(a3!) checkpoint" in schema and "SymInt k, SymInt wpb) -> ()" in schema


def test_the_cmake_target_builds_the_same_library(tmp_path):
    """CMakeLists.txt and spear_amd/csrc/build.py are two recipes for one library: the CMake-built file must
    export every symbol the header declares, at the ABI version the package expects."""
    cmake, ninja = shutil.which("cmake"), shutil.which("ninja")
    clang = "/opt/rocm/lib/llvm/bin/clang++"
    if not (cmake and ninja and os.path.exists(clang)):
        pytest.skip("needs cmake, ninja and the ROCm clang")
    from test_capi_symbols import PROBE_HEADER, declared_functions

    from spear_amd import _btp

    build = tmp_path / "build"
    cfg = [cmake, "-S", ROOT, "-B", str(build), "-G", "Ninja", f"-DCMAKE_HIP_COMPILER={clang}", "-DSPEAR_BTP_TORCH_BINDING=OFF"]
    subprocess.run(cfg, check=True, capture_output=True, timeout=300)
    subprocess.run([cmake, "--build", str(build), "-j8"], check=True, capture_output=True, timeout=600)
    built = build / "libspear_btp.so"
    assert built.exists()
    assert not (build / "_btp_ext.so").exists()  # switched off above: the C-ABI library needs no PyTorch
    lib = ctypes.CDLL(str(built))
    for name in declared_functions() + declared_functions(PROBE_HEADER):
        assert hasattr(lib, name), f"{name} missing from the CMake-built library"
    lib.spear_btp_abi_version.restype = ctypes.c_int
    assert lib.spear_btp_abi_version() == _btp._ABI_VERSION
    # and it validates like the other one
    lib.spear_btp_last_error.restype = ctypes.c_char_p
    assert lib.spear_btp_forward(None, None, None, None, 1, 1, 24, 2, 0, 0, 0, None) == -1
    assert b"multiple of 16" in lib.spear_btp_last_error()
