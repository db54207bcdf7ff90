"""ctypes binding of oracle/brute_force.c (float64 triple loops).  TEST
INFRASTRUCTURE ONLY — see the header of brute_force.c."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libtrittention_brute.so")


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "brute_force.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libtrittention_brute.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def _load():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.trittention_brute.restype = ctypes.c_int
    return _lib


def brute(variant, q, k1, k2, v1, v2, d_out, alpha, causal, windows):
    """One head, numpy float64 [T, D] arrays.  ``variant`` 0 = triple-dot
    (windows = (k1_window, k2_window, kk_left, kk_right)), 1 = dot-product-sum
    (windows = (k_diff,)).  Returns (z, lse, dq, dk1, dk2, dv1, dv2)."""
    lib = _load()
    arrs = [np.ascontiguousarray(a, dtype=np.float64) for a in (q, k1, k2, v1, v2, d_out)]
    T, D = arrs[0].shape
    outs = [np.zeros((T, D)) for _ in range(6)]
    lse = np.zeros(T)
    w = (ctypes.c_int * 4)(*(list(windows) + [0] * (4 - len(windows))))
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    rc = lib.trittention_brute(ctypes.c_int(variant), *[p(a) for a in arrs],
                               ctypes.c_int(T), ctypes.c_int(D), ctypes.c_double(alpha),
                               ctypes.c_int(int(causal)), w, p(outs[0]), p(lse),
                               *[p(a) for a in outs[1:]])
    if rc != 0:
        raise MemoryError("trittention_brute failed")
    return (outs[0], lse, *outs[1:])
