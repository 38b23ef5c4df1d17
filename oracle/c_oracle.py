"""ctypes loader for the C oracle (oracle/q4_oracle.c).  Test infrastructure only."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libq4oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "_build/libq4oracle.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        vp, i = ctypes.c_void_p, ctypes.c_int
        L.q4o_dequant_v2.argtypes = [vp, vp, vp, vp, vp, i, i, i]
        L.q4o_dequant_v2.restype = None
        L.q4o_matmul.argtypes = [vp, vp, vp, i, i, i]
        L.q4o_matmul.restype = None
        L.q4o_matmul_t.argtypes = [vp, vp, vp, i, i, i]
        L.q4o_matmul_t.restype = None
        L.q4o_dequant_table.argtypes = [vp, i, vp]
        L.q4o_dequant_table.restype = None
        L.q4o_dequant_scalar.argtypes = [ctypes.c_uint16, i, i]
        L.q4o_dequant_scalar.restype = ctypes.c_uint16
        L.q4o_f32_to_f16.argtypes = [ctypes.c_float]
        L.q4o_f32_to_f16.restype = ctypes.c_uint16
        L.q4o_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.q4o_f16_to_f32.restype = ctypes.c_float
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def dequant_v2(qweight, qzeros, scales, g_idx) -> np.ndarray:
    qweight = np.ascontiguousarray(qweight, dtype=np.int32)
    qzeros = np.ascontiguousarray(qzeros, dtype=np.int32)
    scales = np.ascontiguousarray(scales, dtype=np.float16)
    g_idx = np.ascontiguousarray(g_idx, dtype=np.int32)
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    out = np.empty((K, N), dtype=np.float16)
    lib().q4o_dequant_v2(_p(qweight), _p(qzeros), _p(scales), _p(g_idx), _p(out), K, N, scales.shape[0])
    return out


def matmul(x, W) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float16)
    W = np.ascontiguousarray(W, dtype=np.float16)
    M, K = x.shape
    N = W.shape[1]
    y = np.empty((M, N), dtype=np.float32)
    lib().q4o_matmul(_p(x), _p(W), _p(y), M, K, N)
    return y


def matmul_t(dy, W) -> np.ndarray:
    dy = np.ascontiguousarray(dy, dtype=np.float16)
    W = np.ascontiguousarray(W, dtype=np.float16)
    M, N = dy.shape
    K = W.shape[0]
    dx = np.empty((M, K), dtype=np.float32)
    lib().q4o_matmul_t(_p(dy), _p(W), _p(dx), M, K, N)
    return dx


def dequant_table(scale_bits) -> np.ndarray:
    sb = np.ascontiguousarray(scale_bits, dtype=np.uint16)
    out = np.empty((sb.size, 16, 16), dtype=np.uint16)
    lib().q4o_dequant_table(_p(sb), sb.size, _p(out))
    return out
