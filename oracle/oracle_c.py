"""ctypes loader for the C oracle (`oq_oracle.c`).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
from pathlib import Path

import numpy as np

_SO = Path(__file__).resolve().parent / "liboq_oracle.so"
_lib = None

_u8p = ctypes.POINTER(ctypes.c_uint8)
_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int32)
_i8p = ctypes.POINTER(ctypes.c_int8)


def lib():
    global _lib
    if _lib is None:
        if not _SO.exists():
            from oracle.build import build_oracle

            build_oracle()
        _lib = ctypes.CDLL(str(_SO))
        _lib.oqo_max_threads.restype = ctypes.c_int
    return _lib


def _ptr(arr, typ):
    return arr.ctypes.data_as(typ) if arr is not None else None


def max_threads() -> int:
    return int(lib().oqo_max_threads())


def rotate_quantize(x32, perm, signs, boundaries, block, eps, inv_sqrt_block, threads=0):
    x32 = np.ascontiguousarray(x32, dtype=np.float32)
    m, k = x32.shape
    perm = np.ascontiguousarray(perm, dtype=np.int32)
    signs = np.ascontiguousarray(signs, dtype=np.int8)
    bounds = np.ascontiguousarray(boundaries, dtype=np.float32)
    codes = np.empty((m, k), dtype=np.uint8)
    norms = np.empty(m, dtype=np.float32)
    rc = lib().oqo_rotate_quantize(
        _ptr(x32, _f32p), ctypes.c_int64(m), ctypes.c_int64(k), _ptr(perm, _i32p),
        _ptr(signs, _i8p), _ptr(bounds, _f32p), ctypes.c_int(bounds.size), ctypes.c_int64(block),
        ctypes.c_float(eps), ctypes.c_float(inv_sqrt_block), _ptr(codes, _u8p), _ptr(norms, _f32p),
        ctypes.c_int(threads))
    if rc:
        raise ValueError("oqo_rotate_quantize rejected its arguments")
    return codes, norms


def unpack(packed, bits, count):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty(count, dtype=np.uint8)
    if lib().oqo_unpack(_ptr(packed, _u8p), ctypes.c_int(bits), ctypes.c_int64(count), _ptr(out, _u8p)):
        raise ValueError("oqo_unpack rejected its arguments")
    return out


def matmul_packed_weight(x32, packed, row_norms, centroids, bias, bits, n, threads=0):
    x32 = np.ascontiguousarray(x32, dtype=np.float32)
    m, k = x32.shape
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    row_norms = np.ascontiguousarray(row_norms, dtype=np.float32)
    centroids = np.ascontiguousarray(centroids, dtype=np.float32)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    out = np.empty((m, n), dtype=np.float32)
    rc = lib().oqo_matmul_packed_weight(
        _ptr(x32, _f32p), _ptr(packed, _u8p), _ptr(row_norms, _f32p), _ptr(centroids, _f32p),
        _ptr(bias, _f32p), ctypes.c_int(bits), ctypes.c_int64(m), ctypes.c_int64(n),
        ctypes.c_int64(k), _ptr(out, _f32p), ctypes.c_int(threads))
    if rc:
        raise ValueError("oqo_matmul_packed_weight rejected its arguments")
    return out


def linear_from_codes(codes, s, c_a, packed_w, w_bits, r_w, c_w, bias, n, threads=0):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    m, k = codes.shape
    s = np.ascontiguousarray(s, dtype=np.float32)
    c_a = np.ascontiguousarray(c_a, dtype=np.float32)
    packed_w = np.ascontiguousarray(packed_w, dtype=np.uint8)
    r_w = np.ascontiguousarray(r_w, dtype=np.float32)
    c_w = np.ascontiguousarray(c_w, dtype=np.float32)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    out = np.empty((m, n), dtype=np.float64)
    rc = lib().oqo_linear_from_codes(
        _ptr(codes, _u8p), _ptr(s, _f32p), _ptr(c_a, _f32p), _ptr(packed_w, _u8p),
        ctypes.c_int(w_bits), _ptr(r_w, _f32p), _ptr(c_w, _f32p), _ptr(bias, _f32p),
        ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k), _ptr(out, _f64p),
        ctypes.c_int(threads))
    if rc:
        raise ValueError("oqo_linear_from_codes rejected its arguments")
    return out
