"""Writes jagged_reference_vectors.npz beside this file: input/output vectors of the reference's own
streaming functions for the one behaviour no identity pins -- the state `parallel_jagged` hands over,
in particular when the prompt length is a multiple of the block length (spear/nn/phalanx/inference.py:
327-357) -- and of `step_jagged` continuing from that state.

The reference module is loaded from its source file (it needs only torch; the package's __init__ would
import the CUDA extension) and run in float64 on the CPU, in this container only. Inputs are stored
already rounded to bfloat16 (as float32) so that every consumer sees the same bits.

    python tests/golden/make_jagged_vectors.py [/root/reference]
"""

from __future__ import annotations

import importlib.util
import pathlib
import sys

import numpy as np
import torch


def load_reference(root: str):
    path = pathlib.Path(root) / "spear" / "nn" / "phalanx" / "inference.py"
    spec = importlib.util.spec_from_file_location("_reference_inference", path)
    mod = importlib.util.module_from_spec(spec)
    sys.modules[spec.name] = mod  # dataclasses looks the module up while the class body runs
    spec.loader.exec_module(mod)
    return mod


def bf16_exact(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(torch.float64)


def main() -> None:
    ref = load_reference(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    blob = {}
    # (name, B, H, D, L, block_len, decode steps): full last block, ragged, shorter than a block, other block length
    cases = [("full", 2, 2, 16, 32, 16, 5), ("ragged", 1, 3, 16, 40, 16, 20), ("short", 2, 1, 16, 5, 16, 12),
             ("one_block", 1, 2, 16, 16, 16, 17), ("bl4", 2, 2, 3, 8, 4, 6)]
    for name, B, H, D, L, bl, steps in cases:
        g = torch.Generator().manual_seed(len(name) * 1000 + L)
        T = L + steps
        A = bf16_exact(torch.sigmoid(torch.randn(B, H, T, generator=g)))
        X, C, V = (bf16_exact(torch.randn(B, H, D, T, generator=g)) for _ in range(3))
        Y, st = ref.parallel_jagged(A[..., :L], X[..., :L], C[..., :L], V[..., :L], block_len=bl)
        blob.update({f"{name}.A": A.float().numpy(), f"{name}.X": X.float().numpy(), f"{name}.C": C.float().numpy(),
                     f"{name}.V": V.float().numpy(), f"{name}.meta": np.array([L, bl, steps, st.i]),
                     f"{name}.Y": Y.numpy(), f"{name}.h_loc": st.h_loc.numpy(), f"{name}.r_pref": st.r_pref.numpy(),
                     f"{name}.c_prev_loc": st.c_prev_loc.numpy()})
        ys = []
        for t in range(L, T):
            y, st = ref.step_jagged(A[:, :, t], X[..., t], C[..., t], V[..., t], st)
            ys.append(y.numpy())
        blob[f"{name}.y_steps"] = np.stack(ys, axis=-1)
        blob[f"{name}.final"] = np.concatenate([st.h_loc.numpy().ravel(), st.r_pref.numpy().ravel(),
                                                st.c_prev_loc.numpy().ravel(), [st.i]])
    path = pathlib.Path(__file__).with_name("jagged_reference_vectors.npz")
    np.savez_compressed(path, **blob)
    print(f"wrote {path} ({path.stat().st_size} bytes, {len(blob)} arrays)")


if __name__ == "__main__":
    main()
