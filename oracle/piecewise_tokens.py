"""ctypes loader for oracle/piecewise_tokens.c (test infrastructure only)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "_build", "libpisa_tokens.so")


def _load():
    if not os.path.exists(_LIB):
        subprocess.check_call(["make", "-s", "-C", _HERE])
    lib = ctypes.CDLL(_LIB)
    dp = ctypes.POINTER(ctypes.c_double)
    lp = ctypes.POINTER(ctypes.c_long)
    lib.pisa_tokens.argtypes = [dp, dp, dp, lp, dp, dp] + [ctypes.c_long] * 5 + [ctypes.c_double]
    lib.pisa_tokens.restype = None
    return lib


def pisa_tokens(q, k, v, indices, block_size=64, scale=None):
    """q,k:[T,K] v:[T,V] for ONE head, indices:[NT,NS]; returns o:[T,V] float64."""
    lib = _load()
    q, k, v = (np.ascontiguousarray(a, dtype=np.float64) for a in (q, k, v))
    idx = np.ascontiguousarray(indices, dtype=np.int64)
    T, K = k.shape
    V = v.shape[1]
    NT = -(-T // block_size)
    assert idx.shape[0] == NT and q.shape == k.shape and v.shape[0] == T
    assert idx.min() >= 0 and idx.max() < NT
    scale = K ** -0.5 if scale is None else scale
    o = np.empty((T, V), dtype=np.float64)
    work = np.empty(NT * K + NT * V + K * V, dtype=np.float64)
    dp = ctypes.POINTER(ctypes.c_double)
    lib.pisa_tokens(q.ctypes.data_as(dp), k.ctypes.data_as(dp), v.ctypes.data_as(dp),
                    idx.ctypes.data_as(ctypes.POINTER(ctypes.c_long)), o.ctypes.data_as(dp),
                    work.ctypes.data_as(dp), T, K, V, block_size, idx.shape[1], float(scale))
    return o
