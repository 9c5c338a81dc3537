"""Builds ``spear_amd/libspear_btp.so`` (HIP kernels + C ABI) for gfx950 with hipcc.

Usage: ``python -m spear_amd.csrc.build`` or ``spear_amd.csrc.build.build()`` followed by
``build_extension()`` (``spear_amd/_btp_ext.so``, the compiled torch binding over the C ABI). hipcc
cross-compiles without a GPU present. The CMake targets in the repository root build the same
two files from the same sources.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB_NAME = "libspear_btp.so"
SOURCES = ["btp_scan.hip", "btp_mfma.hip", "btp_fused.hip", "btp_jagged.hip", "btp_capi.hip", "btp_probe.hip"]
HEADERS = ["btp_device.h", "btp_launch.h", "btp_staging.h", os.path.join("..", "..", "include", "spear_btp.h"),
           os.path.join("..", "..", "include", "spear_btp_probe.h")]

# -packed-fp32-ops is switched off on purpose: scalar fp32 code must not be fused into
# v_pk_*_f32 instructions on this hardware pool.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    cand = shutil.which("hipcc") or os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")
    if not os.path.exists(cand):
        raise RuntimeError("hipcc not found; the BTP library can only be built with the ROCm toolchain")
    return cand


def lib_path() -> str:
    return os.path.join(PKG, LIB_NAME)


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, cwd=HERE, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stdout}\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False, extra_flags: list[str] | None = None, out: str | None = None) -> str:
    """One object per source, compiled side by side (the files are independent and the kernels'
    template instances make each take tens of seconds), then one link."""
    out = out or lib_path()
    hipcc, flags = hipcc_path(), [*HIPCC_FLAGS, *(extra_flags or [])]
    with tempfile.TemporaryDirectory(prefix="spear_btp_build_") as tmp:
        objects = [os.path.join(tmp, os.path.splitext(s)[0] + ".o") for s in SOURCES]
        jobs = [[hipcc, *flags, "-c", os.path.join(HERE, s), "-o", o] for s, o in zip(SOURCES, objects)]
        with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1, 8)) as pool:
            list(pool.map(lambda cmd: _run(cmd, verbose), jobs))
        _run([hipcc, *flags, "-shared", "-o", out, *objects], verbose)
    return out


EXT_NAME = "_btp_ext"
EXT_SOURCE = "btp_torch_ext.cpp"


def ext_path() -> str:
    return os.path.join(PKG, EXT_NAME + ".so")


def build_extension(verbose: bool = False, out: str | None = None) -> str:
    """``spear_amd/_btp_ext.so``: the compiled torch binding over the C ABI (host code only, no kernels),
    linked against ``libspear_btp.so`` beside it. Needs the library built first."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    out = out or ext_path()
    if not os.path.exists(lib_path()):
        raise RuntimeError(f"{lib_path()} is missing; build the C-ABI library before its torch binding")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    includes = [*cpp_extension.include_paths(), sysconfig.get_paths()["include"], os.path.join(rocm, "include")]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [
        hipcc_path(), "-x", "c++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-command-line-argument",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-DTORCH_EXTENSION_NAME={EXT_NAME}", "-DTORCH_API_INCLUDE_EXTENSION_H",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        *[f"-I{p}" for p in includes], os.path.join(HERE, EXT_SOURCE), "-o", out,
        f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
        f"-L{PKG}", "-lspear_btp", "-Wl,-rpath,$ORIGIN",
    ]
    _run(cmd, verbose)
    return out


def is_stale() -> bool:
    out = lib_path()
    if not os.path.exists(out):
        return True
    t = os.path.getmtime(out)
    deps = [os.path.join(HERE, p) for p in SOURCES + HEADERS]
    return any(os.path.getmtime(p) > t for p in deps)


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_extension(verbose=True))
