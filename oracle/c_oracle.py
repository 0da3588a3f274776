"""ctypes loader for the plain-C oracle (oracle/w8a8_oracle.c). TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libw8a8_oracle.so")


def build() -> str:
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _SO


_LIB = None


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        u8, f32, i64, i32 = ctypes.c_uint8, ctypes.c_float, ctypes.c_int64, ctypes.c_int
        P = ctypes.c_void_p
        for name in ("oracle_e4m3fn_decode", "oracle_e5m2_decode"):
            getattr(L, name).argtypes = [u8]
            getattr(L, name).restype = f32
        for name in ("oracle_e4m3fn_encode", "oracle_e5m2_encode",
                     "oracle_e4m3fn_encode_sat", "oracle_e5m2_encode_sat"):
            getattr(L, name).argtypes = [f32]
            getattr(L, name).restype = u8
        L.oracle_fp8_quantize.argtypes = [P, P, f32, i64, i32, i32]
        L.oracle_fp8_quantize.restype = f32
        L.oracle_fp8_gemm_f32.argtypes = [P, P, P, i64, i64, i64, i32]
        L.oracle_fp8_gemm_f32.restype = None
        L.oracle_fp8_gemm_block128_f32.argtypes = [P, P, P, P, P, i64, i64, i64]
        L.oracle_fp8_gemm_block128_f32.restype = None
        L.oracle_int8_gemm_i32.argtypes = [P, P, P, i64, i64, i64]
        L.oracle_int8_gemm_i32.restype = None
        L.oracle_int8_quantize_rows.argtypes = [P, P, P, i64, i64]
        L.oracle_int8_quantize_rows.restype = None
        _LIB = L
    return _LIB


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def fp8_quantize(x_bf16_bits: np.ndarray, scale: float, fmt: int, saturate: bool):
    x = np.ascontiguousarray(x_bf16_bits, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.uint8)
    amax = lib().oracle_fp8_quantize(_p(x), _p(out), scale, x.size, fmt, int(saturate))
    return out, amax


def fp8_gemm_f32(a: np.ndarray, b: np.ndarray, fmt: int = 0) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    m, k = a.shape
    n = b.shape[0]
    c = np.empty((m, n), dtype=np.float32)
    lib().oracle_fp8_gemm_f32(_p(a), _p(b), _p(c), m, n, k, fmt)
    return c


def fp8_gemm_block128_f32(a, b, sa, sb) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    sa = np.ascontiguousarray(sa, dtype=np.float32)
    sb = np.ascontiguousarray(sb, dtype=np.float32)
    m, k = a.shape
    n = b.shape[0]
    c = np.empty((m, n), dtype=np.float32)
    lib().oracle_fp8_gemm_block128_f32(_p(a), _p(b), _p(sa), _p(sb), _p(c), m, n, k)
    return c


def int8_gemm_i32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.int8)
    b = np.ascontiguousarray(b, dtype=np.int8)
    m, k = a.shape
    n = b.shape[0]
    c = np.empty((m, n), dtype=np.int32)
    lib().oracle_int8_gemm_i32(_p(a), _p(b), _p(c), m, n, k)
    return c


def int8_quantize_rows(x_bf16_bits: np.ndarray):
    x = np.ascontiguousarray(x_bf16_bits, dtype=np.uint16)
    rows, k = x.shape
    q = np.empty((rows, k), dtype=np.int8)
    s = np.empty((rows,), dtype=np.float32)
    lib().oracle_int8_quantize_rows(_p(x), _p(q), _p(s), rows, k)
    return q, s
