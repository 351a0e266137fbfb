"""ctypes loader for oracle/libmxfp6_oracle.so (the plain-C oracle).  TEST INFRASTRUCTURE, NOT PRODUCT."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmxfp6_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libmxfp6_oracle.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        u8p, f32p, f64p, u16p = (ctypes.POINTER(t) for t in (ctypes.c_uint8, ctypes.c_float, ctypes.c_double, ctypes.c_uint16))
        L.mxfp6o_decode.restype = ctypes.c_float
        L.mxfp6o_decode.argtypes = [ctypes.c_int, ctypes.c_int]
        L.mxfp6o_e8m0.restype = ctypes.c_float
        L.mxfp6o_e8m0.argtypes = [ctypes.c_int]
        L.mxfp6o_decode_table.argtypes = [ctypes.c_int, f32p]
        L.mxfp6o_quantise.argtypes = [f32p, ctypes.c_long, ctypes.c_long, ctypes.c_int, u8p, u8p]
        L.mxfp6o_dequantise.argtypes = [u8p, u8p, ctypes.c_long, ctypes.c_long, ctypes.c_int, f32p, ctypes.c_int]
        L.mxfp6o_f32_to_bf16.restype = ctypes.c_uint16
        L.mxfp6o_f32_to_bf16.argtypes = [ctypes.c_float]
        gemm_args = [u8p, u8p, u8p, u8p]
        tail = [ctypes.c_long, ctypes.c_long, ctypes.c_long, ctypes.c_int, ctypes.c_int]
        L.mxfp6o_gemm_f32.argtypes = gemm_args + [f32p] + tail
        L.mxfp6o_gemm_bf16.argtypes = gemm_args + [u16p] + tail
        L.mxfp6o_gemm_f64_naive.argtypes = gemm_args + [f64p] + tail
        L.mxfp6o_num_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def _p(a, t):
    return a.ctypes.data_as(ctypes.POINTER(t))


def decode_table(fmt):
    out = np.zeros(64, np.float32)
    lib().mxfp6o_decode_table(fmt, _p(out, ctypes.c_float))
    return out


def quantise(x, fmt):
    x = np.ascontiguousarray(x, np.float32)
    rows, K = x.shape
    packed = np.zeros((rows, K // 4 * 3), np.uint8)
    scales = np.zeros((rows, K // 32), np.uint8)
    rc = lib().mxfp6o_quantise(_p(x, ctypes.c_float), rows, K, fmt, _p(packed, ctypes.c_uint8), _p(scales, ctypes.c_uint8))
    if rc:
        raise ValueError(f"mxfp6o_quantise rc={rc}")
    return packed, scales


def dequantise(packed, scales, fmt, transpose=False):
    packed = np.ascontiguousarray(packed, np.uint8)
    scales = np.ascontiguousarray(scales, np.uint8)
    rows, K = packed.shape[0], packed.shape[1] // 3 * 4
    out = np.zeros((K, rows) if transpose else (rows, K), np.float32)
    rc = lib().mxfp6o_dequantise(_p(packed, ctypes.c_uint8), _p(scales, ctypes.c_uint8), rows, K, fmt, _p(out, ctypes.c_float), int(transpose))
    if rc:
        raise ValueError(f"mxfp6o_dequantise rc={rc}")
    return out


def _gemm(fn, ctype, dtype, ap, bp, asc, bsc, fmt_a, fmt_b):
    ap, bp, asc, bsc = (np.ascontiguousarray(t, np.uint8) for t in (ap, bp, asc, bsc))
    M, N, K = ap.shape[0], bp.shape[0], ap.shape[1] // 3 * 4
    C = np.zeros((M, N), dtype)
    rc = fn(_p(ap, ctypes.c_uint8), _p(bp, ctypes.c_uint8), _p(asc, ctypes.c_uint8), _p(bsc, ctypes.c_uint8), _p(C, ctype), M, N, K, fmt_a, fmt_b)
    if rc:
        raise ValueError(f"oracle gemm rc={rc}")
    return C


def gemm_f32(ap, bp, asc, bsc, fmt_a=2, fmt_b=2):
    return _gemm(lib().mxfp6o_gemm_f32, ctypes.c_float, np.float32, ap, bp, asc, bsc, fmt_a, fmt_b)


def gemm_bf16_bits(ap, bp, asc, bsc, fmt_a=2, fmt_b=2):
    return _gemm(lib().mxfp6o_gemm_bf16, ctypes.c_uint16, np.uint16, ap, bp, asc, bsc, fmt_a, fmt_b)


def gemm_f64_naive(ap, bp, asc, bsc, fmt_a=2, fmt_b=2):
    return _gemm(lib().mxfp6o_gemm_f64_naive, ctypes.c_double, np.float64, ap, bp, asc, bsc, fmt_a, fmt_b)


def num_threads():
    return lib().mxfp6o_num_threads()
