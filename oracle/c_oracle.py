"""ctypes loader for the C restatement of the oracle.  TEST INFRASTRUCTURE ONLY.

Loads oracle/libafir_oracle.so (built by oracle/Makefile).  Used by tests to
cross-check the numpy oracle and by the benchmark's CPU-baseline leg.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libafir_oracle.so")
_lib = None

_DT = {"f16": 0, "bf16": 1, "f32": 2, "i8": 3, "i32": 4, "i64": 5}


def build():
    subprocess.run(["make", "-s", "-C", _HERE], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_f16_to_f32.restype = ctypes.c_float
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.oracle_bf16_to_f32.restype = ctypes.c_float
        L.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.oracle_max_threads.restype = ctypes.c_int
        L.oracle_gather_scale_shift_f16.restype = ctypes.c_int
        L.oracle_compare.restype = ctypes.c_size_t
        _lib = L
    return _lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _sz(v):
    return ctypes.c_size_t(int(v))


def threads() -> int:
    return int(lib().oracle_max_threads())


def add_mul_f32(a, b):
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    out = np.empty_like(a)
    lib().oracle_add_mul_f32(_p(a), _p(b), _p(out), _sz(a.size))
    return out


def bcast_add_rowsum_f32(x, bias):
    x = np.ascontiguousarray(x, np.float32)
    bias = np.ascontiguousarray(bias, np.float32)
    m, n = x.shape
    y = np.empty((m,), np.float32)
    buf = np.empty((threads(), n), np.float32)
    lib().oracle_bcast_add_rowsum_f32(_p(x), _p(bias), _p(y), _sz(m), _sz(n),
                                      _p(buf), ctypes.c_int(threads()))
    return y


def relu_bcast_add_transpose_f16(x, c):
    x = np.ascontiguousarray(x, np.float16)
    c = np.ascontiguousarray(c, np.float16)
    nb, m, n = x.shape
    out = np.empty((nb, n, m), np.float16)
    lib().oracle_relu_bcast_add_transpose_f16(_p(x), _p(c), _p(out), _sz(nb),
                                              _sz(m), _sz(n))
    return out


def gather_scale_shift_f16(table, idx, scale, shift):
    table = np.ascontiguousarray(table, np.float16)
    idx = np.ascontiguousarray(idx, np.int32)
    scale = np.ascontiguousarray(scale, np.float16)
    shift = np.ascontiguousarray(shift, np.float16)
    rows, dim = table.shape
    out = np.empty((idx.size, dim), np.float16)
    bad = lib().oracle_gather_scale_shift_f16(
        _p(table), _p(idx), _p(scale), _p(shift), _p(out), _sz(rows),
        _sz(dim), _sz(idx.size))
    if bad:
        raise IndexError("gather index out of range")
    return out


def matmul_bias_leakyrelu_bf16(a_bits, b_bits, bias_bits, alpha=0.01):
    a = np.ascontiguousarray(a_bits, np.uint16)
    b = np.ascontiguousarray(b_bits, np.uint16)
    bias = np.ascontiguousarray(bias_bits, np.uint16)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2 and bias.size == n
    out = np.empty((m, n), np.uint16)
    buf = np.empty((threads(), n), np.float32)
    lib().oracle_matmul_bias_leakyrelu_bf16(
        _p(a), _p(b), _p(bias), _p(out), _sz(m), _sz(k), _sz(n),
        ctypes.c_float(alpha), _p(buf))
    return out


def compare(actual, expected, dtype, atol, rtol):
    a = np.ascontiguousarray(actual)
    e = np.ascontiguousarray(expected)
    assert a.nbytes == e.nbytes
    mx = ctypes.c_double()
    tot = ctypes.c_double()
    n = a.size
    bad = lib().oracle_compare(_p(a), _p(e), _sz(n), ctypes.c_int(_DT[dtype]),
                               ctypes.c_double(atol), ctypes.c_double(rtol),
                               ctypes.byref(mx), ctypes.byref(tot))
    return {"mismatches": int(bad), "max_abs_diff": mx.value,
            "mean_abs_diff": (tot.value / n) if n else 0.0,
            "passed": bad == 0}
