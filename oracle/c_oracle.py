"""ctypes + numpy front end of ``libf8oracle.so`` (test infrastructure only).

Tensors cross as numpy arrays: bf16/fp16 as uint16 bit patterns, fp32 as
float32, fp8 payloads as uint8.
"""
import ctypes as C
import os

import numpy as np

from . import build as _build

BF16, FP16, FP32 = 0, 1, 2
E4M3FN, E5M2 = 0, 1

_lib = None


def lib():
    global _lib
    if _lib is None:
        path = _build.LIB
        if not os.path.exists(path):
            path = _build.build()
        L = C.CDLL(path)
        L.f8o_bf16_to_f32.restype = C.c_float
        L.f8o_bf16_to_f32.argtypes = [C.c_uint16]
        L.f8o_f32_to_bf16.restype = C.c_uint16
        L.f8o_f32_to_bf16.argtypes = [C.c_float]
        L.f8o_fp16_to_f32.restype = C.c_float
        L.f8o_fp16_to_f32.argtypes = [C.c_uint16]
        L.f8o_f32_to_fp16.restype = C.c_uint16
        L.f8o_f32_to_fp16.argtypes = [C.c_float]
        L.f8o_f32_to_fp8.restype = C.c_uint8
        L.f8o_f32_to_fp8.argtypes = [C.c_float, C.c_int]
        L.f8o_fp8_to_f32.restype = C.c_float
        L.f8o_fp8_to_f32.argtypes = [C.c_uint8, C.c_int]
        L.f8o_f32_to_fp8_n.restype = None
        L.f8o_f32_to_fp8_n.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        L.f8o_fp8_to_f32_n.restype = None
        L.f8o_fp8_to_f32_n.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        L.f8o_amax.restype = C.c_float
        L.f8o_amax.argtypes = [C.c_void_p, C.c_size_t, C.c_int]
        L.f8o_amax_to_scale.restype = C.c_float
        L.f8o_amax_to_scale.argtypes = [C.c_float, C.c_int, C.c_int, C.c_int]
        L.f8o_cast_one.restype = C.c_uint8
        L.f8o_cast_one.argtypes = [C.c_float, C.c_float, C.c_int, C.c_int]
        L.f8o_cast.restype = None
        L.f8o_cast.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int, C.c_float, C.c_int,
                               C.c_int, C.c_void_p, C.c_void_p]
        L.f8o_gemm_emulated.restype = None
        L.f8o_gemm_emulated.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.c_float, C.c_void_p, C.c_int,
                                        C.c_size_t, C.c_float, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int,
                                        C.c_void_p]
        L.f8o_sync_entry.restype = C.c_float
        L.f8o_sync_entry.argtypes = [C.c_float, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int]
        L.f8o_delayed_init.restype = C.c_float
        L.f8o_delayed_init.argtypes = [C.c_float, C.c_void_p, C.c_int, C.c_int, C.c_int]
        _lib = L
    return _lib


def _dtype_code(a: np.ndarray, dtype: int) -> int:
    if dtype in (BF16, FP16):
        assert a.dtype == np.uint16, "bf16/fp16 cross as uint16 bit patterns"
    else:
        assert a.dtype == np.float32
    return dtype


def amax(x: np.ndarray, dtype: int) -> float:
    x = np.ascontiguousarray(x)
    _dtype_code(x, dtype)
    return float(lib().f8o_amax(x.ctypes.data, x.size, dtype))


def amax_to_scale(amax_val: float, math_dtype: int, fp8_fmt: int, orig_is_fp16: bool = False) -> np.float32:
    return np.float32(lib().f8o_amax_to_scale(np.float32(amax_val), math_dtype, fp8_fmt, int(orig_is_fp16)))


def cast(x: np.ndarray, dtype: int, scale, product_dtype: int, fp8_fmt: int, transpose: bool = False):
    """x: 2-D array [rows, cols].  Returns (out[rows,cols], out_t[cols,rows] or None) uint8."""
    assert x.ndim == 2
    x = np.ascontiguousarray(x)
    _dtype_code(x, dtype)
    rows, cols = x.shape
    out = np.empty((rows, cols), np.uint8)
    out_t = np.empty((cols, rows), np.uint8) if transpose else None
    lib().f8o_cast(x.ctypes.data, rows, cols, cols, dtype, np.float32(scale), product_dtype, fp8_fmt,
                   out.ctypes.data, out_t.ctypes.data if transpose else None)
    return out, out_t


def f32_to_fp8(x: np.ndarray, fp8_fmt: int) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32).reshape(-1)
    out = np.empty(x.size, np.uint8)
    lib().f8o_f32_to_fp8_n(x.ctypes.data, x.size, fp8_fmt, out.ctypes.data)
    return out


def fp8_to_f32(codes: np.ndarray, fp8_fmt: int) -> np.ndarray:
    codes = np.ascontiguousarray(codes, np.uint8).reshape(-1)
    out = np.empty(codes.size, np.float32)
    lib().f8o_fp8_to_f32_n(codes.ctypes.data, codes.size, fp8_fmt, out.ctypes.data)
    return out


def gemm_emulated(a: np.ndarray, a_fmt: int, sa, bt: np.ndarray, b_fmt: int, sb, out_dtype: int = BF16):
    """a: uint8 [m,k]; bt: uint8 [n,k] (B transposed).  Returns float32 [m,n] rounded to out_dtype."""
    a = np.ascontiguousarray(a, np.uint8)
    bt = np.ascontiguousarray(bt, np.uint8)
    m, k = a.shape
    n, k2 = bt.shape
    assert k == k2
    out = np.empty((m, n), np.float32)
    lib().f8o_gemm_emulated(a.ctypes.data, a_fmt, k, np.float32(sa), bt.ctypes.data, b_fmt, k, np.float32(sb), m, n,
                            k, out_dtype, out.ctypes.data)
    return out


def sync_entry(amax_val, history: np.ndarray, fp8_fmt: int, orig_is_fp16=False, writeback=False) -> np.float32:
    assert history.dtype == np.float32 and history.flags.c_contiguous
    return np.float32(lib().f8o_sync_entry(np.float32(amax_val), history.ctypes.data, history.size, fp8_fmt,
                                           int(orig_is_fp16), int(writeback)))


def delayed_init(amax_val, history: np.ndarray, fp8_fmt: int, orig_is_fp16=False) -> np.float32:
    assert history.dtype == np.float32 and history.flags.c_contiguous
    return np.float32(lib().f8o_delayed_init(np.float32(amax_val), history.ctypes.data, history.size, fp8_fmt,
                                             int(orig_is_fp16)))
