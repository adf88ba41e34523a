"""Writes tests/golden/attention_small.npz.

The reference holds no golden vectors for this path (its one check,
test.py:42-45, compares against inputs drawn from the GPU RNG and stores
nothing), so these fixtures are produced here: hand-listed, RNG-free inputs
pushed through the fp64 brute-force C loops in oracle/attention_bruteforce.c.
Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle.bruteforce import attention_bruteforce  # noqa: E402


def pattern(shape, a, b, m):
    """Deterministic fp16-exact values in [-1, 1]: ((a*i + b) mod m) / m * 2 - 1 on a 1/64 grid."""
    n = int(np.prod(shape))
    i = np.arange(n, dtype=np.int64)
    x = ((a * i + b) % m).astype(np.float64) / m * 2.0 - 1.0
    return (np.round(x * 64) / 64).reshape(shape)


CASES = [  # name, B, N, H, D, scale, causal
    ("n32_d64_causal", 1, 32, 2, 64, 0.125, 1),
    ("n32_d64_full", 1, 32, 2, 64, 0.125, 0),
    ("n96_d128_causal", 1, 96, 1, 128, 128 ** -0.5, 1),
    ("n64_d128_full", 1, 64, 1, 128, 0.1, 0),
]

if __name__ == "__main__":
    blobs = {}
    for name, B, N, H, D, scale, causal in CASES:
        shape = (B, N, H, D)
        q = pattern(shape, 37, 11, 257)
        k = pattern(shape, 53, 5, 263)
        v = pattern(shape, 29, 3, 269)
        do = pattern(shape, 41, 7, 271)
        out, lse, dq, dk, dv = attention_bruteforce(q, k, v, do, scale, causal)
        for key, val in dict(q=q, k=k, v=v, dout=do).items():
            blobs[f"{name}/{key}"] = val.astype(np.float16)
        for key, val in dict(out=out, lse=lse, dq=dq, dk=dk, dv=dv).items():
            blobs[f"{name}/{key}"] = val.astype(np.float32)
        blobs[f"{name}/meta"] = np.array([B, N, H, D, causal], dtype=np.int64)
        blobs[f"{name}/scale"] = np.array([scale], dtype=np.float64)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "attention_small.npz")
    np.savez_compressed(path, **blobs)
    print("wrote", path, os.path.getsize(path), "bytes")
