"""ctypes loader for oracle/libduo_ref.so (the C restatement).  Test infrastructure only."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build() -> str:
    subprocess.check_call(["make", "-s", "-C", _HERE, "libduo_ref.so"])
    return os.path.join(_HERE, "libduo_ref.so")


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libduo_ref.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _f(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def fwd(q1, k1, v1, cu_q1, cu_k1, q2, k2, v2, pos_q2, pos_k2, cu_q2, cu_k2, scale):
    q1, k1, v1, q2, k2, v2 = map(_f, (q1, k1, v1, q2, k2, v2))
    cu_q1, cu_k1, pos_q2, pos_k2, cu_q2, cu_k2 = map(_i, (cu_q1, cu_k1, pos_q2, pos_k2, cu_q2, cu_k2))
    Hq, D = q1.shape[1], q1.shape[2]
    Hkv = k1.shape[1]
    o1 = np.zeros_like(q1)
    o2 = np.zeros_like(q2)
    lse1 = np.zeros((Hq, q1.shape[0]), np.float32)
    lse2 = np.zeros((Hq, q2.shape[0]), np.float32)
    rc = lib().duo_ref_fwd(_p(q1), _p(k1), _p(v1), _p(cu_q1), _p(cu_k1), _p(q2), _p(k2), _p(v2),
                           _p(pos_q2), _p(pos_k2), _p(cu_q2), _p(cu_k2),
                           ctypes.c_int(len(cu_q1) - 1), ctypes.c_int(Hq), ctypes.c_int(Hkv),
                           ctypes.c_int(D), ctypes.c_float(scale), _p(o1), _p(lse1), _p(o2), _p(lse2))
    if rc != 0:
        raise RuntimeError(f"duo_ref_fwd failed: {rc}")
    return o1, lse1, o2, lse2


def bwd(q1, k1, v1, cu_q1, cu_k1, q2, k2, v2, pos_q2, pos_k2, cu_q2, cu_k2, scale, do1, do2):
    q1, k1, v1, q2, k2, v2, do1, do2 = map(_f, (q1, k1, v1, q2, k2, v2, do1, do2))
    cu_q1, cu_k1, pos_q2, pos_k2, cu_q2, cu_k2 = map(_i, (cu_q1, cu_k1, pos_q2, pos_k2, cu_q2, cu_k2))
    Hq, D = q1.shape[1], q1.shape[2]
    Hkv = k1.shape[1]
    outs = [np.zeros_like(x) for x in (q1, k1, v1, q2, k2, v2)]
    rc = lib().duo_ref_bwd(_p(q1), _p(k1), _p(v1), _p(cu_q1), _p(cu_k1), _p(q2), _p(k2), _p(v2),
                           _p(pos_q2), _p(pos_k2), _p(cu_q2), _p(cu_k2),
                           ctypes.c_int(len(cu_q1) - 1), ctypes.c_int(Hq), ctypes.c_int(Hkv),
                           ctypes.c_int(D), ctypes.c_float(scale), _p(do1), _p(do2),
                           *[_p(x) for x in outs])
    if rc != 0:
        raise RuntimeError(f"duo_ref_bwd failed: {rc}")
    return tuple(outs)


def hard_index(mask):
    m = np.ascontiguousarray(mask, dtype=np.uint8)
    B, S = m.shape
    idx = np.zeros(max(int(m.sum()), 1), np.int32)
    cu = np.zeros(B + 1, np.int32)
    n = lib().duo_ref_hard_index(_p(m), ctypes.c_int(B), ctypes.c_int(S), _p(idx), _p(cu))
    return idx[:n], cu
