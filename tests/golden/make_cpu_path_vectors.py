"""Writes cpu_path_reference_vectors.npz beside this file: outputs of the reference's CPU path
(spear/ops/btp/reference.py: block_two_pass_log / _linspace / _ref) in the dtypes the layer uses, and
the float64 gradients its harness compares kernels with.

What the mathematics pins about these functions is checked elsewhere against the float64 oracle; what
it cannot pin is the exact sequence of roundings of the bfloat16 path (log -> repeat -> masked_fill ->
cumsum -> exp -> einsum, all in bfloat16, reference.py:38-52,119-136), which is what "the CPU reference
path in bf16" of the benchmark's first configuration produces. These vectors record it, so that this
package's restatement can be held to bit equality. The reference module is loaded from its source file
(torch and einops only) and run on the CPU, in this container only.

    python tests/golden/make_cpu_path_vectors.py [/root/reference]
"""

from __future__ import annotations

import importlib.util
import pathlib
import sys

import numpy as np
import torch


def load_reference(root: str):
    path = pathlib.Path(root) / "spear" / "ops" / "btp" / "reference.py"
    spec = importlib.util.spec_from_file_location("_reference_btp_reference", path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[spec.name] = mod
    spec.loader.exec_module(mod)
    return mod


def main() -> None:
    ref = load_reference(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    torch.set_num_threads(1)  # one summation order
    g = torch.Generator().manual_seed(20250101)
    B, H, L = 2, 3, 64
    a = torch.sigmoid(torch.randn(B, H, L, generator=g)).to(torch.bfloat16)
    x = torch.randn(B, H, 16, L, generator=g).to(torch.bfloat16)
    blob = {"a": a.float().numpy(), "x": x.float().numpy()}
    for name, fn in (("log", ref.block_two_pass_log), ("linspace", ref.block_two_pass_linspace)):
        blob[f"{name}.bf16"] = fn(a, x, 16).float().numpy()
        blob[f"{name}.f32"] = fn(a.float(), x.float(), 16).numpy()
    blob["ref.f64"] = ref.block_two_pass_ref(a.double(), x.double()).numpy()
    # gradients the way the reference's harness takes them (spear/ops/btp/runners.py:152-164): autograd
    # through the float64 path, upstream gradient rounded to bfloat16
    dy = torch.randn(B, H, 16, L, generator=g).to(torch.bfloat16)
    a64, x64 = a.double().requires_grad_(True), x.double().requires_grad_(True)
    ref.block_two_pass_ref(a64, x64).backward(dy.double())
    blob.update({"dy": dy.float().numpy(), "ref.f64.dx": x64.grad.numpy(), "ref.f64.dA": a64.grad.numpy()})
    path = pathlib.Path(__file__).with_name("cpu_path_reference_vectors.npz")
    np.savez_compressed(path, **blob)
    print(f"wrote {path} ({path.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
