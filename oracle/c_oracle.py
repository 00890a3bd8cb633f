"""ctypes wrapper over oracle/quik_oracle.c (test infrastructure only)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libquik_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-s", "-C", _HERE, "libquik_oracle.so"], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.qo_half_to_float.restype = ctypes.c_float
        _lib.qo_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.qo_double_to_half.restype = ctypes.c_uint16
        _lib.qo_double_to_half.argtypes = [ctypes.c_double]
        _lib.qo_float_to_bf16.restype = ctypes.c_uint16
        _lib.qo_float_to_bf16.argtypes = [ctypes.c_float]
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _i64(v):
    return ctypes.c_int64(int(v))


def asym_quantize(x_bits, int_idx, fp_idx, bits, is_bf16=False):
    """x_bits: uint16 [M, in] storage bit patterns.  Returns (dst, meta_bits, fp_bits)."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    int_idx = np.ascontiguousarray(int_idx, dtype=np.int64)
    fp_idx = np.ascontiguousarray(fp_idx, dtype=np.int64)
    M, cols = x_bits.shape
    K, F = int_idx.size, fp_idx.size
    dst = np.zeros((M, K // 2 if bits == 4 else K), dtype=np.uint8)
    meta = np.zeros(2 * M, dtype=np.uint16)
    fp_x = np.zeros((M, F), dtype=np.uint16)
    lib().qo_asym_quantize(_p(x_bits), _i64(M), _i64(cols), _p(int_idx), _i64(K), _p(fp_idx), _i64(F),
                           ctypes.c_int(bits), ctypes.c_int(int(is_bf16)), _p(dst), _p(meta), _p(fp_x))
    if bits == 8:
        dst = dst.view(np.int8)
    return dst, meta, fp_x


def int4_matmul(a, b):
    a = np.ascontiguousarray(a, np.uint8)
    b = np.ascontiguousarray(b, np.uint8)
    M, N, K = a.shape[0], b.shape[0], a.shape[1] * 2
    c = np.zeros((M, N), np.int32)
    lib().qo_int4_matmul(_p(a), _p(b), _p(c), _i64(M), _i64(N), _i64(K))
    return c


def int8_matmul(a, b):
    a = np.ascontiguousarray(a, np.int8)
    b = np.ascontiguousarray(b, np.int8)
    M, N, K = a.shape[0], b.shape[0], a.shape[1]
    c = np.zeros((M, N), np.int32)
    lib().qo_int8_matmul(_p(a), _p(b), _p(c), _i64(M), _i64(N), _i64(K))
    return c


def asym_dequantize(acc, meta_bits, scol_bits, wred_bits, y_bits, bits, is_bf16=False):
    acc = np.ascontiguousarray(acc, np.int32)
    rows, cols = acc.shape
    out = np.zeros((rows, cols), np.uint16)
    args = [np.ascontiguousarray(a, np.uint16) for a in (meta_bits, scol_bits, wred_bits, y_bits)]
    lib().qo_asym_dequantize(_p(acc), _p(args[0]), _p(args[1]), _p(args[2]), _p(args[3]), _i64(rows), _i64(cols),
                             ctypes.c_int(bits), ctypes.c_int(int(is_bf16)), _p(out))
    return out


def sym_quantize(x_bits, scale_bits, bits):
    x_bits = np.ascontiguousarray(x_bits, np.uint16)
    scale_bits = np.ascontiguousarray(scale_bits, np.uint16)
    rows, cols = x_bits.shape
    dst = np.zeros((rows, (cols + 1) // 2 if bits == 4 else cols), np.uint8)
    lib().qo_sym_quantize(_p(x_bits), _p(scale_bits), _i64(rows), _i64(cols), ctypes.c_int(bits), _p(dst))
    return dst.view(np.int8) if bits == 8 else dst


def sym_dequantize(x, kind, srow_bits, scol_bits, y_bits):
    if kind == 8:
        x = np.ascontiguousarray(x, np.int8)
    elif kind == 16:
        x = np.ascontiguousarray(x, np.uint16)
    else:
        x = np.ascontiguousarray(x, np.int32)
    rows, cols = x.shape
    out = np.zeros((rows, cols), np.uint16)
    a = [np.ascontiguousarray(v, np.uint16) for v in (srow_bits, scol_bits, y_bits)]
    lib().qo_sym_dequantize(_p(x), ctypes.c_int(kind), _p(a[0]), _p(a[1]), _p(a[2]), _i64(rows), _i64(cols), _p(out))
    return out
