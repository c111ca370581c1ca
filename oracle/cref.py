"""TEST INFRASTRUCTURE ONLY -- ctypes front end of liboracle.so (the plain-C restatement).

Built by ``make -C oracle`` (``__graft_entry__.build()`` does it); the tests build it on
demand when gcc is present.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-s", "-B"], check=True)
    return os.path.join(_HERE, "liboracle.so")


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _i64(x):
    return ctypes.c_int64(int(x))


def unpack_u4(wp: np.ndarray) -> np.ndarray:
    wp = np.ascontiguousarray(wp, dtype=np.uint8)
    N, K = wp.shape[0], wp.shape[1] * 2
    out = np.empty((N, K), dtype=np.int8)
    lib().orc_unpack_u4(_p(wp), _p(out), _i64(N), _i64(K))
    return out


def convert_s4(wp: np.ndarray) -> np.ndarray:
    wp = np.ascontiguousarray(wp, dtype=np.uint8)
    N, K = wp.shape[0], wp.shape[1] * 2
    out = np.empty((N, K), dtype=np.int8)
    lib().orc_convert_s4(_p(wp), _p(out), _i64(N), _i64(K))
    return out


def dequant_w4(wp, scales_bits, zeros_bits, zero_scalar, group, kind) -> np.ndarray:
    """scales_bits / zeros_bits: uint16 bit patterns [N, K/group] or None.  Returns uint16 bits."""
    wp = np.ascontiguousarray(wp, dtype=np.uint8)
    N, K = wp.shape[0], wp.shape[1] * 2
    out = np.empty((N, K), dtype=np.uint16)
    s = None if scales_bits is None else np.ascontiguousarray(scales_bits, dtype=np.uint16)
    z = None if zeros_bits is None else np.ascontiguousarray(zeros_bits, dtype=np.uint16)
    lib().orc_dequant_w4(_p(wp), _p(s), _p(z), ctypes.c_double(zero_scalar), _p(out), _i64(N), _i64(K), _i64(group),
                         ctypes.c_int(kind))
    return out


def gemm_w4a16(a_bits, w_bits, kind, out_kind) -> np.ndarray:
    a = np.ascontiguousarray(a_bits, dtype=np.uint16)
    w = np.ascontiguousarray(w_bits, dtype=np.uint16)
    M, K = a.shape
    N = w.shape[0]
    out = np.empty((M, N), dtype=np.float32 if out_kind == 2 else np.uint16)
    lib().orc_gemm_w4a16(_p(a), _p(w), _p(out), _i64(M), _i64(N), _i64(K), ctypes.c_int(kind), ctypes.c_int(out_kind))
    return out


def gemm_i8(a, b, b_layout) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.int8)
    b = np.ascontiguousarray(b, dtype=np.int8)
    M, K = a.shape
    N = b.shape[0] if b_layout else b.shape[1]
    out = np.empty((M, N), dtype=np.int32)
    lib().orc_gemm_i8(_p(a), _p(b), _p(out), _i64(M), _i64(N), _i64(K), ctypes.c_int(b_layout))
    return out


def rescale(acc, sa, sb, out_kind) -> np.ndarray:
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    M, N = acc.shape
    sa = None if sa is None else np.ascontiguousarray(sa, dtype=np.float32)
    sb = None if sb is None else np.ascontiguousarray(sb, dtype=np.float32)
    out = np.empty((M, N), dtype=np.float32 if out_kind == 2 else np.uint16)
    lib().orc_rescale(_p(acc), _p(sa), _p(sb), _i64(0 if sb is None else sb.size), _p(out), _i64(M), _i64(N),
                      ctypes.c_int(out_kind))
    return out


def act_quant(x: np.ndarray, round_scale: bool = False):
    """x float32 [M,N] -> (int8 [M,N], float32 [M])."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, N = x.shape
    y = np.empty((M, N), dtype=np.int8)
    s = np.empty(M, dtype=np.float32)
    lib().orc_act_quant(_p(x), _p(y), _p(s), _i64(M), _i64(N), ctypes.c_int(int(round_scale)))
    return y, s


def act_quant_quotient_check(n: int, seed: int = 0):
    """(pairs whose rounded integer differs, pairs whose raw quotient differs) between x / s and
    the reciprocal-and-two-fma quotient, over n pseudo-random pairs."""
    f = lib().orc_act_quant_quotient_check
    f.restype = ctypes.c_int64
    bad_q = ctypes.c_int64(0)
    bad_int = f(_i64(n), ctypes.c_uint64(seed), ctypes.byref(bad_q))
    return int(bad_int), int(bad_q.value)
