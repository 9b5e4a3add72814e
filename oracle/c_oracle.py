"""ctypes wrapper of the scalar C restatement (oracle/fp8_ref.c).  TEST INFRASTRUCTURE ONLY.

``build()`` compiles it with gcc; the arrays are numpy (uint16 views of bf16 in, uint8 / float32 out).
"""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import c_float, c_int, c_int64, c_uint8, c_void_p
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
SRC = HERE / "fp8_ref.c"
LIB = HERE / "libfp8ref.so"

_lib = None


def build() -> Path:
    cmd = ["gcc", "-O2", "-fPIC", "-shared", "-ffp-contract=off", "-o", str(LIB), str(SRC), "-lm"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"gcc failed on {SRC}:\n{res.stderr}")
    return LIB


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB.exists():
            build()
        lib = ctypes.CDLL(str(LIB))
        lib.fp8ref_e4m3_from_f32.restype = c_uint8
        lib.fp8ref_e4m3_from_f32.argtypes = [c_float]
        lib.fp8ref_e4m3_to_f32.restype = c_float
        lib.fp8ref_e4m3_to_f32.argtypes = [c_uint8]
        lib.fp8ref_quant_rowwise.argtypes = [c_void_p, c_int64, c_int64, c_void_p, c_void_p]
        lib.fp8ref_bf16_from_f32.restype = ctypes.c_uint16
        lib.fp8ref_bf16_from_f32.argtypes = [c_float]
        lib.fp8ref_quant_rowwise_f32.argtypes = [c_void_p, c_int64, c_int64, c_void_p, c_void_p]
        lib.fp8ref_exp32.restype = c_float
        lib.fp8ref_exp32.argtypes = [c_float]
        lib.fp8ref_silu32.restype = c_float
        lib.fp8ref_silu32.argtypes = [c_float]
        lib.fp8ref_swiglu.argtypes = [c_void_p, c_void_p, c_int64, c_void_p]
        lib.fp8ref_combine_rows.argtypes = [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]
        lib.fp8ref_combine_rows.restype = None
        lib.fp8ref_quant_tensorwise.argtypes = [c_void_p, c_int64, c_void_p, c_void_p]
        lib.fp8ref_quant_block128.argtypes = [c_void_p, c_int64, c_int64, c_void_p, c_void_p]
        lib.fp8ref_quant_group128.argtypes = [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int]
        lib.fp8ref_check_fast_div.restype = c_int64
        lib.fp8ref_check_fast_div.argtypes = [c_void_p, c_int64, c_void_p]
        _lib = lib
    return _lib


def _u16(x: np.ndarray) -> np.ndarray:
    assert x.dtype == np.uint16
    return np.ascontiguousarray(x)


def bf16_from_f32(v: float) -> int:
    return int(load().fp8ref_bf16_from_f32(v))


def quant_rowwise_f32(x_f32: np.ndarray):
    assert x_f32.dtype == np.float32
    x = np.ascontiguousarray(x_f32)
    R, C = x.shape
    q = np.empty((R, C), np.uint8)
    s = np.empty((R, 1), np.float32)
    load().fp8ref_quant_rowwise_f32(x.ctypes.data, R, C, q.ctypes.data, s.ctypes.data)
    return q, s


def swiglu(g_u16: np.ndarray, u_u16: np.ndarray) -> np.ndarray:
    """bf16(bf16(silu(g)) * u) on uint16 views of bf16 arrays of equal shape."""
    g, u = _u16(g_u16), _u16(u_u16)
    assert g.shape == u.shape
    h = np.empty(g.shape, np.uint16)
    load().fp8ref_swiglu(g.ctypes.data, u.ctypes.data, g.size, h.ctypes.data)
    return h


def swiglu_quant_group128(g_u16: np.ndarray, u_u16: np.ndarray):
    return quant_group128(swiglu(g_u16, u_u16), mode=0)


def combine_rows(rows_u16: np.ndarray, row_map: np.ndarray, weights: np.ndarray, mode: int = 0) -> np.ndarray:
    """out[t] = sum_s weights[t, s] * rows[row_map[t, s]] (slot order; < 0 skipped).  weights: uint16 view
    of bf16, or float32 (mode 1 only).  mode 0: bf16 rounding at every step; 1: fp32 fma accumulator."""
    rows = _u16(rows_u16)
    rm = np.ascontiguousarray(row_map, dtype=np.int32)
    T, topk = rm.shape
    w = np.ascontiguousarray(weights)
    assert w.shape == rm.shape and w.dtype in (np.uint16, np.float32)
    out = np.empty((T, rows.shape[1]), np.uint16)
    w16 = w.ctypes.data if w.dtype == np.uint16 else None
    w32 = w.ctypes.data if w.dtype == np.float32 else None
    load().fp8ref_combine_rows(rows.ctypes.data, rows.shape[1], rm.ctypes.data, w16, w32, T, topk, mode, out.ctypes.data)
    return out


def quant_rowwise(x_u16: np.ndarray):
    x = _u16(x_u16)
    R, C = x.shape
    q = np.empty((R, C), np.uint8)
    s = np.empty((R, 1), np.float32)
    load().fp8ref_quant_rowwise(x.ctypes.data, R, C, q.ctypes.data, s.ctypes.data)
    return q, s


def quant_tensorwise(x_u16: np.ndarray):
    x = _u16(x_u16)
    q = np.empty(x.shape, np.uint8)
    s = np.empty(1, np.float32)
    load().fp8ref_quant_tensorwise(x.ctypes.data, x.size, q.ctypes.data, s.ctypes.data)
    return q, s


def quant_block128(x_u16: np.ndarray):
    x = _u16(x_u16)
    R, C = x.shape
    q = np.empty((R, C), np.uint8)
    s = np.empty((-(-R // 128), -(-C // 128)), np.float32)
    load().fp8ref_quant_block128(x.ctypes.data, R, C, q.ctypes.data, s.ctypes.data)
    return q, s


def quant_group128(x_u16: np.ndarray, mode: int = 0):
    x = _u16(x_u16)
    M, K = x.shape
    q = np.empty((M, K), np.uint8)
    s = np.empty((M, -(-K // 128)), np.float32)
    load().fp8ref_quant_group128(x.ctypes.data, M, K, q.ctypes.data, s.ctypes.data, mode)
    return q, s


def check_fast_div(scales_f32: np.ndarray):
    """(bad byte count, fp32 mismatches with |x/s| >= 2^-11) over all 65536 bf16 x per scale."""
    s = np.ascontiguousarray(scales_f32, dtype=np.float32)
    soft = ctypes.c_int64(0)
    bad = load().fp8ref_check_fast_div(s.ctypes.data, s.size, ctypes.byref(soft))
    return int(bad), int(soft.value)
