"""Writes tests/golden/attention_small.npz.

The reference (nightly-Rust only) cannot be run, so these vectors do not come
from it: inputs are seeded, expected outputs are a float64 two-pass
softmax(scale * q.K^T + causal mask).V computed here with numpy, independent of
both the oracle and the HIP kernels.  They pin the oracle against drift and are
small enough to commit.

    python tests/golden/make_golden.py
"""
import os

import numpy as np


def brute_force(q, k, v, scale, position_index):
    """q [S,B,Hq,D], k/v [B,Hkv,cap,D] (float64) -> out [S,B,Hq,D], lse [S,B,Hq]."""
    S, B, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    out = np.zeros_like(q)
    lse = np.zeros((S, B, Hq))
    for t in range(S):
        n = position_index + t + 1
        for b in range(B):
            for h in range(Hq):
                s = (k[b, h // G, :n] @ q[t, b, h]) * scale
                m = s.max()
                e = np.exp(s - m)
                out[t, b, h] = (e / e.sum()) @ v[b, h // G, :n]
                lse[t, b, h] = m + np.log(e.sum())
    return out, lse


def main():
    rng = np.random.default_rng(20240607)
    cases = {}
    for name, (S, B, Hq, Hkv, cap, p0) in {
        "mha": (5, 2, 4, 4, 16, 0),
        "gqa": (7, 1, 8, 2, 24, 9),
        "mqa_decode": (1, 3, 6, 1, 40, 33),
    }.items():
        D = 128
        # values on the binary16 grid so every storage type holds them exactly enough
        q = rng.standard_normal((S, B, Hq, D)).astype(np.float16)
        k = rng.standard_normal((B, Hkv, cap, D)).astype(np.float16)
        v = rng.standard_normal((B, Hkv, cap, D)).astype(np.float16)
        scale = 1.0 / np.sqrt(D)
        out, lse = brute_force(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64),
                               scale, p0)
        cases[name + "_q"] = q
        cases[name + "_k"] = k
        cases[name + "_v"] = v
        cases[name + "_out"] = out.astype(np.float32)
        cases[name + "_lse"] = lse.astype(np.float32)
        cases[name + "_p0"] = np.int64(p0)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "attention_small.npz")
    np.savez_compressed(path, **cases)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
