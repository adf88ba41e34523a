"""ctypes binding of the fp64 brute-force C loops.  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libattention_bruteforce.so")


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "libattention_bruteforce.so"])


def _load():
    if not os.path.exists(_LIB):
        build()
    lib = ctypes.CDLL(_LIB)
    dp = ctypes.POINTER(ctypes.c_double)
    lib.attention_bruteforce.argtypes = [dp] * 9 + [ctypes.c_int] * 4 + [ctypes.c_double, ctypes.c_int]
    lib.attention_bruteforce.restype = ctypes.c_int
    return lib


def attention_bruteforce(q, k, v, dout, scale, causal):
    """q, k, v, dout: array-likes of shape (B, N, H, D).  Returns float64 numpy
    arrays (out, lse, dq, dk, dv); lse is (B, H, N)."""
    lib = _load()
    q, k, v, dout = (np.ascontiguousarray(np.asarray(t, dtype=np.float64)) for t in (q, k, v, dout))
    B, N, H, D = q.shape
    out, dq, dk, dv = (np.empty_like(q) for _ in range(4))
    lse = np.empty((B, H, N), dtype=np.float64)
    ptr = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))
    rc = lib.attention_bruteforce(ptr(q), ptr(k), ptr(v), ptr(dout), ptr(out), ptr(lse), ptr(dq), ptr(dk), ptr(dv),
                                  B, N, H, D, float(scale), int(bool(causal)))
    if rc != 0:
        raise MemoryError("attention_bruteforce: allocation failed")
    return out, lse, dq, dk, dv
