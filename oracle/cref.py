"""ctypes binding of the scalar C oracle (oracle/awq_ref.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libawq_oracle.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-s", "-B", "-C", _HERE, "libawq_oracle.so"], check=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.awqref_moe_align.restype = ctypes.c_long
        L.awqref_f2h.restype = ctypes.c_uint16
        L.awqref_f2h.argtypes = [ctypes.c_float]
        L.awqref_h2f.restype = ctypes.c_float
        L.awqref_h2f.argtypes = [ctypes.c_uint16]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def unpack(words: np.ndarray) -> np.ndarray:
    w = np.ascontiguousarray(words, dtype=np.int32)
    out = np.empty((w.shape[0], w.shape[1] * 8), np.uint8)
    lib().awqref_unpack(_p(w), _p(out), ctypes.c_long(w.shape[0]), ctypes.c_long(w.shape[1]))
    return out


def dequantize(qweight, scales, qzeros, group: int) -> np.ndarray:
    qw = np.ascontiguousarray(qweight, dtype=np.int32)
    sc = np.ascontiguousarray(scales, dtype=np.float16)
    qz = np.ascontiguousarray(qzeros, dtype=np.int32)
    K, N = qw.shape[0], qw.shape[1] * 8
    if group <= 0:
        group = K
    out = np.empty((K, N), np.float16)
    lib().awqref_dequantize(_p(qw), _p(sc), _p(qz), _p(out), ctypes.c_long(K), ctypes.c_long(N),
                            ctypes.c_long(group))
    return out


def gemm(x, qweight, scales, qzeros, group: int):
    """Returns (fp16 [M,N], float64 [M,N])."""
    xx = np.ascontiguousarray(x, dtype=np.float16)
    qw = np.ascontiguousarray(qweight, dtype=np.int32)
    sc = np.ascontiguousarray(scales, dtype=np.float16)
    qz = np.ascontiguousarray(qzeros, dtype=np.int32)
    M, K, N = xx.shape[0], qw.shape[0], qw.shape[1] * 8
    if group <= 0:
        group = K
    y = np.empty((M, N), np.float16)
    yw = np.empty((M, N), np.float64)
    lib().awqref_gemm(_p(xx), _p(qw), _p(sc), _p(qz), _p(y), _p(yw), ctypes.c_long(M),
                      ctypes.c_long(K), ctypes.c_long(N), ctypes.c_long(group))
    return y, yw


def moe_align(topk_ids, num_experts: int, tile_m: int):
    ids = np.ascontiguousarray(topk_ids, dtype=np.int32).reshape(-1)
    n = ids.size
    cap = n + num_experts * (tile_m - 1)
    sorted_ids = np.empty(max(cap, 1), np.int32)
    expert_ids = np.empty(max(cap // tile_m + 1, 1), np.int32)
    npad = lib().awqref_moe_align(_p(ids), ctypes.c_long(n), ctypes.c_long(num_experts),
                                  ctypes.c_long(tile_m), _p(sorted_ids), _p(expert_ids))
    return sorted_ids[:npad].copy(), expert_ids[:npad // tile_m].copy(), int(npad)
