"""ctypes loader for oracle/brute.c (test infrastructure only)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "_build", "libbrute.so")


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE])


def _load():
    if not os.path.exists(_LIB):
        build()
    lib = ctypes.CDLL(_LIB)
    dp = ctypes.POINTER(ctypes.c_double)
    lib.brute_linear_attn.argtypes = [dp, dp, dp, dp, dp, dp, ctypes.c_long, ctypes.c_long,
                                      ctypes.c_long, ctypes.c_double, ctypes.c_double, ctypes.c_int]
    lib.brute_linear_attn.restype = None
    return lib


def brute_linear_attn(q, k, v, scale, eps=1e-6, normalize=True, q_rope=None, k_rope=None):
    """q,k:[L,DK] v:[L,DV] for ONE head; returns o:[L,DV] float64."""
    lib = _load()
    q = np.ascontiguousarray(q, dtype=np.float64)
    k = np.ascontiguousarray(k, dtype=np.float64)
    v = np.ascontiguousarray(v, dtype=np.float64)
    qn = q if q_rope is None else np.ascontiguousarray(q_rope, dtype=np.float64)
    kn = k if k_rope is None else np.ascontiguousarray(k_rope, dtype=np.float64)
    L, DK = q.shape
    DV = v.shape[1]
    o = np.empty((L, DV), dtype=np.float64)
    dp = ctypes.POINTER(ctypes.c_double)
    lib.brute_linear_attn(q.ctypes.data_as(dp), k.ctypes.data_as(dp), qn.ctypes.data_as(dp),
                          kn.ctypes.data_as(dp), v.ctypes.data_as(dp), o.ctypes.data_as(dp),
                          L, DK, DV, float(scale), float(eps), int(bool(normalize)))
    return o
