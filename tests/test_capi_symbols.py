"""The C-ABI library loads without a GPU and exports exactly what include/spear_btp.h declares."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "spear_btp.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(spear_(?:btp|phalanx)_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    assert declared_functions() == [
        "spear_btp_abi_version",
        "spear_btp_backward",
        "spear_btp_backward_loggate",
        "spear_btp_copy",
        "spear_btp_forward",
        "spear_btp_forward_loggate",
        "spear_btp_last_error",
        "spear_phalanx_mix_backward",
        "spear_phalanx_mix_forward",
    ]


def test_library_exports_every_declared_symbol():
    from spear_amd import _btp

    path = _btp.library_path()
    if not os.path.exists(path):
        pytest.fail(f"{path} is not built; run `python -m spear_amd.csrc.build`")
    lib = ctypes.CDLL(path)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} missing from {path}"


def test_constants_match_the_header():
    from spear_amd import _btp

    text = open(HEADER).read()
    defs = dict(re.findall(r"#define\s+(SPEAR_BTP_\w+)\s+\(?(-?0x[0-9a-fA-F]+|-?\d+)u?\)?", text))
    assert int(defs["SPEAR_BTP_BF16"]) == _btp._BF16
    assert int(defs["SPEAR_BTP_F16"]) == _btp._F16
    assert int(defs["SPEAR_BTP_F32"]) == _btp._F32
    assert int(defs["SPEAR_BTP_WRITE_CHECKPOINT"], 16) == _btp.FLAG_WRITE_CHECKPOINT
    assert int(defs["SPEAR_BTP_PATH_MFMA"], 16) == _btp.FLAG_PATH_MFMA


def test_host_side_validation_needs_no_gpu():
    """Argument errors are reported through the return code and spear_btp_last_error()."""
    from spear_amd import _btp

    lib = _btp.load_library()
    assert lib.spear_btp_abi_version() == 5
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p -= p % 16
    p += 16
    # L not a multiple of 16
    assert lib.spear_btp_forward(p, p, p, None, 1, 1, 24, 2, 0, 0, 0, None) == -1
    assert b"multiple of 16" in lib.spear_btp_last_error()
    # bad k
    assert lib.spear_btp_forward(p, p, p, None, 1, 1, 32, 3, 0, 0, 0, None) == -1
    assert b"k must be 1 or 2" in lib.spear_btp_last_error()
    # fp32 inputs are not accepted
    assert lib.spear_btp_forward(p, p, p, None, 1, 1, 32, 2, 2, 2, 0, None) == -1
    assert b"float16 or bfloat16" in lib.spear_btp_last_error()
    # y neither fp32 nor the input dtype
    assert lib.spear_btp_forward(p, p, p, None, 1, 1, 32, 2, 0, 1, 0, None) == -1
    # NULL tensors
    assert lib.spear_btp_forward(None, p, p, None, 1, 1, 32, 2, 0, 0, 0, None) == -2
    assert lib.spear_btp_backward(p, p, p, None, None, p, 1, 1, 32, 2, 0, 0, 0, None) == -2
    # checkpoint requested but not supplied
    assert lib.spear_btp_forward(p, p, p, None, 1, 1, 32, 2, 0, 0, 1, None) == -2
    # misaligned pointer
    assert lib.spear_btp_forward(p + 2, p, p, None, 1, 1, 32, 2, 0, 0, 0, None) == -1
    assert b"aligned" in lib.spear_btp_last_error()
    # unknown flag
    assert lib.spear_btp_backward(p, p, p, None, p, p, 1, 1, 32, 2, 0, 0, 0x80, None) == -1
    # empty problem is a successful no-op and clears the error string
    assert lib.spear_btp_forward(p, p, p, None, 0, 4, 32, 2, 0, 0, 0, None) == 0
    assert lib.spear_btp_last_error() == b""
    assert lib.spear_btp_copy(p, p, 24, None) == -1
