"""ctypes view of oracle/libdaxq_oracle_c.so (bit-level closed forms).

TEST INFRASTRUCTURE ONLY.  Used by tests/ to pin oracle/daxq_oracle.py.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libdaxq_oracle_c.so")


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "daxq_oracle_c.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libdaxq_oracle_c.so"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        p, i64, f32 = C.c_void_p, C.c_int64, C.c_float
        L.daxo_act_scale.restype = f32
        L.daxo_act_scale.argtypes = [C.c_uint16, f32]
        L.daxo_f32_to_e4m3fn.restype = C.c_uint8
        L.daxo_f32_to_e4m3fn.argtypes = [f32]
        L.daxo_e4m3fn_to_f32.restype = f32
        L.daxo_e4m3fn_to_f32.argtypes = [C.c_uint8]
        L.daxo_e5m2_to_f32.restype = f32
        L.daxo_e5m2_to_f32.argtypes = [C.c_uint8]
        L.daxo_f32_to_bf16.restype = C.c_uint16
        L.daxo_f32_to_bf16.argtypes = [f32]
        for name, args in {
            "daxo_act_quant_i8": [p, i64, i64, p, p],
            "daxo_act_quant_e4m3": [p, i64, i64, p, p],
            "daxo_act_quant_e5m2": [p, i64, i64, p, p],
            "daxo_f32_to_e5m2_vec": [p, i64, p],
            "daxo_quant_e5m2_vec": [p, i64, f32, p],
            "daxo_weight_scale": [p, i64, i64, f32, p],
            "daxo_gemm_i8": [p, p, i64, i64, i64, p],
            "daxo_epilogue_i8": [p, p, p, p, i64, i64, p],
            "daxo_f32_to_e4m3fn_vec": [p, i64, p],
            "daxo_act_scale_vec": [p, i64, f32, p],
            "daxo_quant_i8_vec": [p, i64, f32, p],
            "daxo_quant_e4m3_vec": [p, i64, f32, p],
        }.items():
            fn = getattr(L, name)
            fn.restype = None
            fn.argtypes = args
        _lib = L
    return _lib


def _ptr(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def act_scale_vec(amax_bits: np.ndarray, qmax: float) -> np.ndarray:
    amax_bits = np.ascontiguousarray(amax_bits, dtype=np.uint16)
    out = np.empty(amax_bits.shape, np.float32)
    lib().daxo_act_scale_vec(_ptr(amax_bits), amax_bits.size, qmax, _ptr(out))
    return out


def f32_to_e4m3fn(v: np.ndarray) -> np.ndarray:
    v = np.ascontiguousarray(v, dtype=np.float32)
    out = np.empty(v.shape, np.uint8)
    lib().daxo_f32_to_e4m3fn_vec(_ptr(v), v.size, _ptr(out))
    return out


def e4m3fn_table() -> np.ndarray:
    return np.array([lib().daxo_e4m3fn_to_f32(b) for b in range(256)], np.float32)


def f32_to_e5m2(v: np.ndarray) -> np.ndarray:
    v = np.ascontiguousarray(v, dtype=np.float32)
    out = np.empty(v.shape, np.uint8)
    lib().daxo_f32_to_e5m2_vec(_ptr(v), v.size, _ptr(out))
    return out


def e5m2_table() -> np.ndarray:
    return np.array([lib().daxo_e5m2_to_f32(b) for b in range(256)], np.float32)


def quant_e5m2_vec(x_bits: np.ndarray, s: float) -> np.ndarray:
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    out = np.empty(x_bits.shape, np.uint8)
    lib().daxo_quant_e5m2_vec(_ptr(x_bits), x_bits.size, s, _ptr(out))
    return out


def act_quant_e5m2(x_bits: np.ndarray):
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    m, k = x_bits.shape
    q = np.empty((m, k), np.uint8)
    s = np.empty((m,), np.float32)
    lib().daxo_act_quant_e5m2(_ptr(x_bits), m, k, _ptr(q), _ptr(s))
    return q, s


def quant_i8_vec(x_bits: np.ndarray, s: float) -> np.ndarray:
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    out = np.empty(x_bits.shape, np.int8)
    lib().daxo_quant_i8_vec(_ptr(x_bits), x_bits.size, s, _ptr(out))
    return out


def quant_e4m3_vec(x_bits: np.ndarray, s: float) -> np.ndarray:
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    out = np.empty(x_bits.shape, np.uint8)
    lib().daxo_quant_e4m3_vec(_ptr(x_bits), x_bits.size, s, _ptr(out))
    return out


def act_quant_i8(x_bits: np.ndarray):
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    m, k = x_bits.shape
    q = np.empty((m, k), np.int8)
    s = np.empty((m,), np.float32)
    lib().daxo_act_quant_i8(_ptr(x_bits), m, k, _ptr(q), _ptr(s))
    return q, s


def act_quant_e4m3(x_bits: np.ndarray):
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    m, k = x_bits.shape
    q = np.empty((m, k), np.uint8)
    s = np.empty((m,), np.float32)
    lib().daxo_act_quant_e4m3(_ptr(x_bits), m, k, _ptr(q), _ptr(s))
    return q, s


def weight_scale(w_bits: np.ndarray, qmax: float) -> np.ndarray:
    w_bits = np.ascontiguousarray(w_bits, dtype=np.uint16)
    n, k = w_bits.shape
    s = np.empty((n,), np.float32)
    lib().daxo_weight_scale(_ptr(w_bits), n, k, qmax, _ptr(s))
    return s


def gemm_i8(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.int8)
    b = np.ascontiguousarray(b, dtype=np.int8)
    m, k = a.shape
    n = b.shape[0]
    c = np.empty((m, n), np.int32)
    lib().daxo_gemm_i8(_ptr(a), _ptr(b), m, n, k, _ptr(c))
    return c


def epilogue_i8(acc, sx, sw, bias_bits) -> np.ndarray:
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    sx = np.ascontiguousarray(sx, dtype=np.float32).reshape(-1)
    sw = np.ascontiguousarray(sw, dtype=np.float32).reshape(-1)
    m, n = acc.shape
    out = np.empty((m, n), np.uint16)
    bp = None
    if bias_bits is not None:
        bias_bits = np.ascontiguousarray(bias_bits, dtype=np.uint16)
        bp = _ptr(bias_bits)
    lib().daxo_epilogue_i8(_ptr(acc), _ptr(sx), _ptr(sw), bp, m, n, _ptr(out))
    return out
