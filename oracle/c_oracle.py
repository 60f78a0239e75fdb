"""ctypes binding of oracle/gmm_oracle.c (test infrastructure only)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libgmm_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []), stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_LIB_PATH)
        lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
        lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        lib.oracle_gmm_w8a8.restype = ctypes.c_int
        lib.oracle_gmm_w8a8.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                        ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                        ctypes.c_void_p]
        lib.oracle_gmm_a16w8_f64.restype = ctypes.c_int
        lib.oracle_gmm_a16w8_f64.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                             ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int64,
                                             ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        _lib = lib
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def f32_to_bf16(v: float) -> int:
    return int(_load().oracle_f32_to_bf16(ctypes.c_float(v)))


def gmm_w8a8(x, w, group_list=None, bias=None, scale=None, per_token=None, *, group_list_type=0, transpose_b=False):
    """Returns (acc_plus_bias int32 [M,N], bf16 bits uint16 [M,N])."""
    x = np.ascontiguousarray(x, dtype=np.int8)
    w = np.ascontiguousarray(w, dtype=np.int8)
    m, k = x.shape
    e = w.shape[0]
    n = w.shape[1] if transpose_b else w.shape[2]
    gl = None if group_list is None else np.ascontiguousarray(group_list, dtype=np.int64)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    scale = None if scale is None else np.ascontiguousarray(scale, dtype=np.float32)
    per_token = None if per_token is None else np.ascontiguousarray(per_token, dtype=np.float32)
    acc = np.empty((m, n), dtype=np.int32)
    out = np.empty((m, n), dtype=np.uint16)
    rc = _load().oracle_gmm_w8a8(_ptr(x), _ptr(w), _ptr(gl), int(group_list_type), m, k, n, e, int(transpose_b),
                                 _ptr(bias), _ptr(scale), _ptr(per_token), _ptr(acc), _ptr(out))
    if rc != 0:
        raise ValueError(f"oracle_gmm_w8a8 failed with {rc}")
    return acc, out


def gmm_a16w8_f64(x_bf16_bits, w, scale_bf16_bits, offset_bf16_bits, group_list, *, group_list_type=0):
    x = np.ascontiguousarray(x_bf16_bits, dtype=np.uint16)
    w = np.ascontiguousarray(w, dtype=np.int8)
    m, k = x.shape
    e, _, n = w.shape
    s = None if scale_bf16_bits is None else np.ascontiguousarray(scale_bf16_bits, dtype=np.uint16)
    o = None if offset_bf16_bits is None else np.ascontiguousarray(offset_bf16_bits, dtype=np.uint16)
    gl = None if group_list is None else np.ascontiguousarray(group_list, dtype=np.int64)
    out = np.empty((m, n), dtype=np.float64)
    rc = _load().oracle_gmm_a16w8_f64(_ptr(x), _ptr(w), _ptr(s), _ptr(o), _ptr(gl), int(group_list_type), m, k, n,
                                      e, _ptr(out))
    if rc != 0:
        raise ValueError(f"oracle_gmm_a16w8_f64 failed with {rc}")
    return out
