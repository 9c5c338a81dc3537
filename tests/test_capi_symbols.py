"""The C-ABI library loads without a GPU and exports exactly what include/spear_btp.h (the operator) and
include/spear_btp_probe.h (the measurement aids) declare."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "spear_btp.h")
PROBE_HEADER = os.path.join(ROOT, "include", "spear_btp_probe.h")


def declared_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(spear_(?:btp|phalanx|jagged)_\w+)\s*\(", text)))


def test_measurement_aids_are_declared_apart_from_the_operator():
    assert declared_functions(PROBE_HEADER) == [
        "spear_btp_copy", "spear_btp_stream_probe", "spear_btp_stream_probe_mix", "spear_btp_stream_probe_shape"]
    assert not set(declared_functions(PROBE_HEADER)) & set(declared_functions())


def test_header_declares_the_expected_entry_points():
    assert declared_functions() == [
        "spear_btp_abi_version",
        "spear_btp_backward",
        "spear_btp_backward_loggate",
        "spear_btp_forward",
        "spear_btp_forward_loggate",
        "spear_btp_last_error",
        "spear_jagged_prefill",
        "spear_jagged_step",
        "spear_phalanx_mix_backward",
        "spear_phalanx_mix_backward_bias",
        "spear_phalanx_mix_backward_ex",
        "spear_phalanx_mix_backward_sum_rows",
        "spear_phalanx_mix_forward",
        "spear_phalanx_mix_prefill",
        "spear_phalanx_mix_step",
    ]


def test_library_exports_every_declared_symbol():
    from spear_amd import _btp

    path = _btp.library_path()
    if not os.path.exists(path):
        pytest.fail(f"{path} is not built; run `python -m spear_amd.csrc.build`")
    lib = ctypes.CDLL(path)
    for name in declared_functions() + declared_functions(PROBE_HEADER):
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
    jag = dict(re.findall(r"#define\s+(SPEAR_JAGGED_\w+)\s+(0x[0-9a-fA-F]+)u", text))
    assert int(jag["SPEAR_JAGGED_LOG_A"], 16) == _btp.FLAG_JAGGED_LOG_A
    assert int(jag["SPEAR_JAGGED_LOG_R"], 16) == _btp.FLAG_JAGGED_LOG_R


def test_host_side_validation_needs_no_gpu():
    """Argument errors are reported through the return code and spear_btp_last_error()."""
    from spear_amd import _btp

    lib = _btp.load_library()
    assert lib.spear_btp_abi_version() == _btp._ABI_VERSION
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
    assert lib.spear_btp_stream_probe(p, None, p, 100, None) == -1
    # fused layer kernels: a batch row must fit one 32-bit buffer resource
    assert lib.spear_phalanx_mix_forward(p, p, p, p, p, 1, 1 << 20, 128, 128, 0, 0, None) == -1
    assert b"below 2 GiB" in lib.spear_btp_last_error()
    # SPEAR_MIX_QKV_GATE (0x1) and SPEAR_MIX_F32_RESULTS (0x2) are the flags of the fused entry points
    for bad in (0x4, 0x8, 0x10):
        assert lib.spear_phalanx_mix_forward(p, p, p, p, p, 1, 32, 4, 4, 0, bad, None) == -1
        assert b"unknown flag" in lib.spear_btp_last_error()
        assert lib.spear_phalanx_mix_backward(p, p, p, p, p, p, p, p, p, 1, 32, 4, 4, 0, bad, None) == -1
        assert b"unknown flag" in lib.spear_btp_last_error()
    # heads must be a multiple of kv_heads, nothing else
    assert lib.spear_phalanx_mix_forward(p, p, p, p, p, 1, 32, 6, 4, 0, 0, None) == -1
    assert b"divisible by kv_heads" in lib.spear_btp_last_error()
    assert lib.spear_phalanx_mix_backward(p, p, p, p, p, p, p, p, p, 1, 32, 6, 4, 0, 0, None) == -1
    assert b"divisible by kv_heads" in lib.spear_btp_last_error()
    assert _btp.FLAG_MIX_QKV_GATE == int(re.search(r"#define SPEAR_MIX_QKV_GATE (0x[0-9a-f]+)u", open(HEADER).read()).group(1), 16)
    # backward with column sums: the three arrays come together and with the row count the library states
    rows = lib.spear_phalanx_mix_backward_sum_rows(2, 64, 8)
    assert lib.spear_phalanx_mix_backward_sum_rows(2, 60, 8) == 0 and lib.spear_phalanx_mix_backward_sum_rows(0, 64, 8) == 0
    # one row per workgroup: 4 blocks of 16 steps of a batch row
    assert rows == 2 and lib.spear_phalanx_mix_backward_sum_rows(3, 80, 8) == 6
    assert lib.spear_phalanx_mix_backward_sum_rows(3, 80, 128) == 6
    sums = lambda sa, sb, sc, n, ld=(0, 0, 0, 0): lib.spear_phalanx_mix_backward_ex(
        p, p, p, p, p, p, p, p, p, *ld, sa, sb, sc, n, 2, 64, 8, 8, 0, 0, None)
    assert sums(p, p, None, rows) == -2
    assert b"given together" in lib.spear_btp_last_error()
    assert sums(p, p, p, rows + 1) == -1
    assert b"rows for this shape" in lib.spear_btp_last_error()
    assert sums(p + 4, p, p, rows) == -1
    assert lib.spear_phalanx_mix_backward_ex(p, p, p, p, p, p, p, p, p, 0, 0, 0, 0, p, p, p, rows, 2, 64, 8, 8, 0, 0x1, None) == -1
    assert b"layer form" in lib.spear_btp_last_error()
    # output row strides: 0 or an even number of elements not below the tensor's width
    assert sums(None, None, None, 0, (4, 0, 0, 0)) == -1
    assert b"row stride" in lib.spear_btp_last_error()
    assert sums(None, None, None, 0, (0, 0, 0, 131)) == -1
    assert sums(None, None, None, 0, (0, 0, 0, 1 << 24)) == -1
    assert b"below 2 GiB" in lib.spear_btp_last_error()


def test_streaming_entry_points_validate_on_the_host():
    from spear_amd import _btp

    lib = _btp.load_library()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p += 16 - p % 16
    pre = lambda *a: lib.spear_jagged_prefill(*a)
    # a, x, c, v, carry, y, h, r, cprev, B, H, D, L, block_len, a_dt, x_dt, state_dt, r_dt, flags, stream
    assert pre(p, p, p, None, None, p, None, None, None, 1, 1, 16, 32, 16, 0, 0, 0, 0, 0, None) == -1
    assert b"c and v must be given together" in lib.spear_btp_last_error()
    assert pre(p, p, None, None, None, p, p, None, None, 1, 1, 16, 32, 16, 0, 0, 0, 0, 0, None) == -1
    assert b"given together" in lib.spear_btp_last_error()
    assert pre(p, p, None, None, None, p, None, None, None, 1, 1, 16, 32, 0, 0, 0, 0, 0, 0, None) == -1
    assert b"block_len must be positive" in lib.spear_btp_last_error()
    assert pre(p, p, None, None, None, p, None, None, None, 1, 1, 16, 32, 16, 1, 0, 0, 0, 0, None) == -1
    assert b"a must be float32 or match x dtype" in lib.spear_btp_last_error()
    assert pre(p, p, None, None, None, p, None, None, None, 1, 1, 16, 32, 16, 0, 0, 1, 0, 0, None) == -1
    assert b"state must be float32 or match x dtype" in lib.spear_btp_last_error()
    assert pre(p, p, None, None, None, p, None, None, None, 1, 1, 16, 32, 16, 0, 0, 0, 0, 0x8, None) == -1
    assert pre(None, p, None, None, None, p, None, None, None, 1, 1, 16, 32, 16, 0, 0, 0, 0, 0, None) == -2
    assert pre(p, p, None, None, None, p, None, None, None, 1, 0, 16, 32, 16, 0, 0, 0, 0, 0, None) == 0
    step = lambda *a: lib.spear_jagged_step(*a)
    # a_t, x_t, c_t, v_t, y_t, h_in, r_in, cp_in, h_out, r_out, cp_out, B, H, D, boundary, dtypes x4, flags, tiny, stream
    assert step(p, p, None, None, p, p, p, p, p, p, None, 1, 1, 16, 1, 0, 0, 0, 0, 0, 0.0, None) == -2  # boundary needs c_prev_out
    assert step(p, p, p, None, p, p, p, p, p, p, p, 1, 1, 16, 0, 0, 0, 0, 0, 0, 0.0, None) == -1
    assert b"c_t and v_t must be given together" in lib.spear_btp_last_error()
    assert step(p, p, None, None, p, p, p, p, p, p, p, 1, 1, 0, 0, 0, 0, 0, 0, 0, 0.0, None) == -1
    assert b"D must be positive" in lib.spear_btp_last_error()
    assert step(p, p, None, None, p, p, p, p, p, p, p, 1, 1, 16, 0, 0, 0, 7, 0, 0, 0.0, None) == -1
    assert step(p, p, None, None, p, p, p, p, p, p, p, 0, 1, 16, 0, 0, 0, 0, 0, 0, 0.0, None) == 0
    assert lib.spear_btp_last_error() == b""
