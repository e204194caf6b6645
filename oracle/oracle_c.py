"""ctypes loader for oracle/liboracle_c.so (the scalar C restatement).

TEST INFRASTRUCTURE ONLY -- see oracle_c.c.  Build with ``make -C oracle``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build() -> str:
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle_c.so"])
    return os.path.join(_HERE, "liboracle_c.so")


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle_c.so")
        if not os.path.exists(path):
            build()
        L = C.CDLL(path)
        L.oc_d2h.restype = C.c_uint16
        L.oc_d2h.argtypes = [C.c_double]
        L.oc_h2d.restype = C.c_double
        L.oc_h2d.argtypes = [C.c_uint16]
        L.oc_dequant.restype = C.c_uint16
        L.oc_dequant.argtypes = [C.c_uint32, C.c_int, C.c_uint16, C.c_uint16]
        L.oc_unpack.restype = None
        L.oc_unpack.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                                C.c_void_p, C.c_void_p]
        L.oc_dequantize.restype = None
        L.oc_dequantize.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                    C.c_int64, C.c_size_t, C.c_size_t, C.c_void_p]
        L.oc_sparse_pack.restype = C.c_int64
        L.oc_sparse_pack.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                     C.c_size_t, C.c_size_t]
        L.oc_matvec.restype = None
        L.oc_matvec.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                C.c_void_p, C.c_int64, C.c_size_t, C.c_size_t, C.c_void_p]
        _LIB = L
    return _LIB


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a).view(dtype)


def unpack(bits, matrix, mask, K):
    m = _c(matrix, np.uint32)
    k = _c(mask, np.uint32)
    S = m.shape[1]
    codes = np.empty((K, S), np.uint8)
    keep = np.empty((K, S), np.uint8)
    lib().oc_unpack(bits, _p(m), _p(k), K, S, _p(codes), _p(keep))
    return codes, keep.astype(bool)


def dequantize(bits, matrix, scales, zeros, group_size, mask, K):
    m = _c(matrix, np.uint32)
    k = _c(mask, np.uint32)
    sc = _c(np.atleast_2d(scales), np.uint16)
    ze = _c(np.atleast_2d(zeros), np.uint16)
    S = m.shape[1]
    out = np.empty((K, S), np.uint16)
    lib().oc_dequantize(bits, _p(m), _p(k), _p(sc), _p(ze), int(group_size), K, S, _p(out))
    return out.view(np.float16)


def sparse_pack(codes_sk, keep_sk):
    codes_sk = np.ascontiguousarray(codes_sk, dtype=np.uint8)
    keep_sk = np.ascontiguousarray(keep_sk, dtype=np.uint8)
    S, K = codes_sk.shape
    wt = np.zeros((K // 16, S), np.uint32)
    msk = np.zeros((K // 32, S), np.uint32)
    bad = lib().oc_sparse_pack(_p(wt), _p(msk), _p(codes_sk), _p(keep_sk), S, K)
    return wt.view(np.int32), msk.view(np.int32), int(bad)


def matvec(bits, matrix, mask, x, scales, zeros, group_size, outs):
    m = _c(matrix, np.uint32)
    k = _c(mask, np.uint32)
    xs = _c(x.reshape(-1), np.uint16)
    sc = _c(np.atleast_2d(scales), np.uint16)
    ze = _c(np.atleast_2d(zeros), np.uint16)
    K, S = xs.shape[0], m.shape[1]
    o = np.ascontiguousarray(outs.reshape(-1)).view(np.uint16).copy()
    lib().oc_matvec(bits, _p(m), _p(k), _p(xs), _p(sc), _p(ze), int(group_size), K, S, _p(o))
    return o.view(np.float16)


def dequant_scalar(v, bits, scale, zero):
    s = int(np.asarray(scale, np.float16).view(np.uint16))
    z = int(np.asarray(zero, np.float16).view(np.uint16))
    r = lib().oc_dequant(int(v), bits, s, z)
    return np.array(r, np.uint16).view(np.float16)
