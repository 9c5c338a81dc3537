"""Writes layer_reference_vectors.npz beside this file: the benchmark's first configuration computed by
the reference's own layer on its CPU path -- ``Phalanx(dim=512, length=128, method="pytorch",
dtype=bfloat16)`` with default initialisation under ``torch.manual_seed(0)``, input
``randn(8, 128, 512).to(bfloat16)`` drawn right after, output ``y [8, 128, 512]``.

Two things about that configuration are conventions rather than mathematics, so only the reference can
pin them: the order in which the layer draws its default weights from the global generator
(spear/nn/phalanx/swr.py:157-164,271) and the rounding sequence of the bfloat16 CPU path. The file holds,
per parameter, its shape, float64 sum and sum of squares and first 8 values; the input's and the output's
sums; and every 8th time step of the output.

The reference's sources are loaded file by file (swr.py and reference.py need only torch and einops); the
packages above them are registered as empty modules because ``spear/__init__.py`` imports the CUDA
extension, which does not exist here. Runs on the CPU, in this container only.

    python tests/golden/make_layer_vectors.py [/root/reference]
"""

from __future__ import annotations

import importlib.util
import pathlib
import sys
import types

import numpy as np
import torch


def load_reference_layer(root: str):
    base = pathlib.Path(root) / "spear"
    for pkg in ("spear", "spear.ops", "spear.ops.btp", "spear.nn", "spear.nn.phalanx"):
        mod = types.ModuleType(pkg)
        mod.__path__ = []  # a package without an __init__ of its own
        sys.modules[pkg] = mod

    def load(name: str, rel: str):
        spec = importlib.util.spec_from_file_location(name, base / rel)
        mod = importlib.util.module_from_spec(spec)
        sys.modules[name] = mod
        spec.loader.exec_module(mod)
        return mod

    load("spear.ops.btp.reference", "ops/btp/reference.py")
    return load("spear.nn.phalanx.swr", "nn/phalanx/swr.py")


def main() -> None:
    swr = load_reference_layer(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    torch.set_num_threads(1)
    torch.manual_seed(0)
    layer = swr.Phalanx(dim=512, length=128, method="pytorch", dtype=torch.bfloat16)
    x = torch.randn(8, 128, 512).to(torch.bfloat16)
    with torch.no_grad():
        y = layer(x)
    blob = {"x.sums": np.array([x.double().sum().item(), x.double().square().sum().item()]),
            "y.sums": np.array([y.double().sum().item(), y.double().square().sum().item()]),
            "y.every8": y[:, ::8, :].float().numpy(), "y.dtype_is_bf16": np.array([y.dtype == torch.bfloat16])}
    for name, p in layer.state_dict().items():
        d = p.double()
        blob[f"param.{name}"] = np.concatenate([[float(n) for n in p.shape] + [0.0] * (2 - p.dim()),
                                                [d.sum().item(), d.square().sum().item()], d.flatten()[:8].numpy()])
    path = pathlib.Path(__file__).with_name("layer_reference_vectors.npz")
    np.savez_compressed(path, **blob)
    print(f"wrote {path} ({path.stat().st_size} bytes); parameters: {[k for k in blob if k.startswith('param.')]}")


if __name__ == "__main__":
    main()
