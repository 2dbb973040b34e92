"""ctypes access to the C restatement under ``oracle/c`` (test infrastructure:
checker and timed CPU baseline only)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(_HERE, "_build", "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force and os.path.exists(LIB):
        os.remove(LIB)
    subprocess.run(["make", "-s", "-C", os.path.join(_HERE, "c")], check=True)
    return LIB


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = ctypes.CDLL(LIB)
        _lib.oracle_threads.restype = ctypes.c_int
        _lib.oracle_double_to_half.restype = ctypes.c_uint16
        _lib.oracle_double_to_half.argtypes = [ctypes.c_double]
        _lib.oracle_half_to_float.restype = ctypes.c_float
        _lib.oracle_half_to_float.argtypes = [ctypes.c_uint16]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def threads() -> int:
    return lib().oracle_threads()


def set_threads(n: int) -> None:
    lib().oracle_set_threads(ctypes.c_int(n))


def dequant(qweight, qzeros, scales, g_idx=None, bits=4, group_size=128):
    per = 32 // bits
    k, n = qweight.shape[0] * per, qweight.shape[1]
    out = np.empty((k, n), np.float16)
    g = None if g_idx is None else np.ascontiguousarray(g_idx, np.int32)
    lib().oracle_gptq_dequant(_p(np.ascontiguousarray(qweight)), _p(np.ascontiguousarray(qzeros)),
                              _p(np.ascontiguousarray(scales)), _p(g), _p(out),
                              ctypes.c_int(n), ctypes.c_int(k), ctypes.c_int(group_size), ctypes.c_int(bits))
    return out


def matmul(x, qweight, qzeros, scales, g_idx=None, bits=4, group_size=128):
    per = 32 // bits
    k, n = qweight.shape[0] * per, qweight.shape[1]
    x2 = np.ascontiguousarray(x.reshape(-1, k))
    m = x2.shape[0]
    y = np.empty((m, n), np.float16)
    g = None if g_idx is None else np.ascontiguousarray(g_idx, np.int32)
    lib().oracle_gptq_matmul(_p(x2), _p(np.ascontiguousarray(qweight)), _p(np.ascontiguousarray(qzeros)),
                             _p(np.ascontiguousarray(scales)), _p(g), _p(y), ctypes.c_int(m),
                             ctypes.c_int(n), ctypes.c_int(k), ctypes.c_int(group_size), ctypes.c_int(bits))
    return y.reshape(*x.shape[:-1], n)
