"""Writes btp_window_vectors.npz beside this file: small known-answer vectors for the BTP op.

The reference ships no data files for this path (its tests compare kernel and Python reference live,
tests/btp/test_numerics.py:126-183), so these vectors are evaluated here from the definition alone:

    y_t   = sum_{s=w(t)}^{t} P(s,t) x_s            P(s,t) = prod_{j=s+1}^{t} a_j
    dx_s  = sum_{t>=s, w(t)<=s} P(s,t) dy_t
    dA_j  = sum_{t>=j} sum_{w(t)<=s<j} (prod_{i=s+1..t, i!=j} a_i) <dy_t, x_s>

with w(t) the first step of the block before t's block (k = 2) or of t's own block (k = 1), which is
what the two passes of spear/ops/btp/reference.py:105-139 compute. Everything is explicit float64
products and sums in plain loops: no recurrence, no decay matrix, no logarithm, no division, and no
code shared with the oracle or the kernels, so that a mistake there cannot hide here.

Inputs are stored already rounded to bfloat16 (as float32), so every consumer sees the same bits.

    python tests/golden/make_vectors.py
"""

from __future__ import annotations

import pathlib

import numpy as np

BLOCK = 16
CHAN = 16


def to_bf16(a: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even to bfloat16, kept as float32."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def window_start(t: int, k: int) -> int:
    return max(0, (t // BLOCK - (k - 1)) * BLOCK)


def closed_form(a: np.ndarray, x: np.ndarray, dy: np.ndarray, k: int):
    """a [L], x [16, L], dy [16, L] (float64) -> y [16, L], dx [16, L], dA [L]."""
    L = a.shape[0]
    y = np.zeros((CHAN, L))
    dx = np.zeros((CHAN, L))
    dA = np.zeros(L)
    for t in range(L):
        for s in range(window_start(t, k), t + 1):
            p = 1.0
            for j in range(s + 1, t + 1):
                p *= a[j]
            y[:, t] += p * x[:, s]
            dx[:, s] += p * dy[:, t]
            w = float(dy[:, t] @ x[:, s])
            for j in range(s + 1, t + 1):
                q = 1.0
                for i in range(s + 1, t + 1):
                    if i != j:
                        q *= a[i]
                dA[j] += q * w
    return y, dx, dA


def cases():
    rng = np.random.RandomState(20240229)
    out = {}
    # smooth gates: sigmoid(N(0,1)), the reference's default sampler (spear/testing/numerics/sampling.py:56-59)
    L = 64
    a = 1.0 / (1.0 + np.exp(-rng.randn(2, L)))
    out["smooth"] = (a, 0.5 * rng.randn(2, CHAN, L), rng.randn(2, CHAN, L))
    # exact zeros, exact ones and tiny values inside and at the edges of blocks; ragged tail of one block
    L = 48
    a = 1.0 / (1.0 + np.exp(-2.0 * rng.randn(2, L)))
    a[0, [0, 15, 16, 17, 31, 40]] = 0.0
    a[0, [5, 32, 47]] = 1.0
    a[1, 16:32] = 1.0
    a[1, [3, 33]] = 1e-6
    out["edges"] = (a, rng.randn(2, CHAN, L), rng.randn(2, CHAN, L))
    # a single block: no carry at all
    L = 16
    out["one_block"] = (rng.uniform(0.2, 1.0, (1, L)), rng.randn(1, CHAN, L), rng.randn(1, CHAN, L))
    return out


def main() -> None:
    blob = {}
    for name, (a, x, dy) in cases().items():
        a, x, dy = to_bf16(a), to_bf16(x), to_bf16(dy)
        blob[f"{name}.coeff"], blob[f"{name}.x"], blob[f"{name}.dy"] = a, x, dy
        for k in (1, 2):
            rows = [closed_form(a[h].astype(np.float64), x[h].astype(np.float64), dy[h].astype(np.float64), k)
                    for h in range(a.shape[0])]
            blob[f"{name}.k{k}.y"] = np.stack([r[0] for r in rows])
            blob[f"{name}.k{k}.dx"] = np.stack([r[1] for r in rows])
            blob[f"{name}.k{k}.dA"] = np.stack([r[2] for r in rows])
    path = pathlib.Path(__file__).with_name("btp_window_vectors.npz")
    np.savez_compressed(path, **blob)
    print(f"wrote {path} ({path.stat().st_size} bytes, {len(blob)} arrays)")


if __name__ == "__main__":
    main()
