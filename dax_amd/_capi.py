"""ctypes binding of the C ABI in include/daxq.h (dax_amd/lib/libdaxq.so).

Loading is lazy and loud: a missing library or a non-gfx950 device raises RuntimeError;
nothing here falls back to another implementation.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdaxq.so")
ABI_VERSION = 5

_lock = threading.Lock()
_lib = None
_checked_devices = set()

_P, _I64, _F32, _INT = C.c_void_p, C.c_int64, C.c_float, C.c_int

# name -> argtypes; every entry point declared in include/daxq.h
SIGNATURES = {
    "daxq_abi_version": [],
    "daxq_last_error": [],
    "daxq_device_info": [_INT, C.POINTER(_INT), C.POINTER(_INT), C.POINTER(_INT), C.c_char_p, _INT],
    "daxq_init": [],
    "daxq_act_quant_i8": [_P, _I64, _I64, _I64, _P, _I64, _P, _P],
    "daxq_act_quant_e4m3": [_P, _I64, _I64, _I64, _P, _I64, _P, _P],
    "daxq_act_quant_e5m2": [_P, _I64, _I64, _I64, _P, _I64, _P, _P],
    "daxq_layernorm_act_quant_i8": [_P, _I64, _I64, _I64, _P, _P, _I64, _F32, _P, _I64, _P, _I64, _P, _P],
    "daxq_layernorm_act_quant_e4m3": [_P, _I64, _I64, _I64, _P, _P, _I64, _F32, _P, _I64, _P, _I64, _P, _P],
    "daxq_layernorm_act_quant_e5m2": [_P, _I64, _I64, _I64, _P, _P, _I64, _F32, _P, _I64, _P, _I64, _P, _P],
    "daxq_gelu_tanh_act_quant_i8": [_P, _I64, _I64, _I64, _P, _I64, _P, _I64, _P, _P],
    "daxq_gelu_tanh_act_quant_e4m3": [_P, _I64, _I64, _I64, _P, _I64, _P, _I64, _P, _P],
    "daxq_gelu_tanh_act_quant_e5m2": [_P, _I64, _I64, _I64, _P, _I64, _P, _I64, _P, _P],
    "daxq_quantize_rows_i8": [_P, _I64, _I64, _I64, _P, _P, _I64, _P],
    "daxq_quantize_rows_e4m3": [_P, _I64, _I64, _I64, _P, _P, _I64, _P],
    "daxq_quantize_rows_e5m2": [_P, _I64, _I64, _I64, _P, _P, _I64, _P],
    "daxq_tensor_scale": [_P, _P, _I64, _F32, _F32, _INT, _P, _P, _I64, _P],
    "daxq_tensor_minmax_update": [_P, _P, _I64, _P, _P, _P],
    "daxq_broadcast_f32": [_P, _P, _I64, _P],
    "daxq_row_minmax": [_P, _I64, _I64, _I64, _P, _P, _P],
    "daxq_row_minmax_t": [_P, _INT, _I64, _I64, _I64, _P, _P, _P],
    "daxq_act_quant_rows": [_P, _INT, _INT, _I64, _I64, _I64, _P, _I64, _P, _P],
    "daxq_act_quant_rows_ex": [_P, _INT, _INT, _I64, _I64, _I64, _P, _I64, _P, _F32, _F32, _INT, _P],
    "daxq_quantize_rows": [_P, _INT, _INT, _I64, _I64, _I64, _P, _P, _I64, _P],
    "daxq_block_scale": [_P, _INT, _INT, C.POINTER(_I64), C.POINTER(C.c_int32), _F32, _F32, _INT, _P, _P],
    "daxq_block_quantize": [_P, _INT, _INT, _INT, C.POINTER(_I64), C.POINTER(C.c_int32), _P, _INT, _P, _P],
    "daxq_scale_from_minmax": [_P, _P, _I64, _F32, _P, _P],
    "daxq_scale_from_minmax_eps": [_P, _P, _I64, _F32, _F32, _P, _P],
    "daxq_linear_i8": [_P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _P, _I64, _I64, _I64, _I64, _P],
    "daxq_linear_e4m3": [_P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _P, _I64, _I64, _I64, _I64, _P],
    "daxq_linear_e5m2_e4m3": [_P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _P, _I64, _I64, _I64, _I64, _P],
    "daxq_linear_splitk_choice": [_I64, _I64, _I64],
    "daxq_linear_tile_order_choice": [_I64, _I64, _I64],
    "daxq_linear_splitk_workspace_bytes": [_I64, _I64, _INT],
    "daxq_linear_w8a8_splitk": [_INT, _INT, _P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _I64, _I64, _I64, _INT, _P, _I64, _P],
    "daxq_linear_w8a8_splitk_static": [_INT, _INT, _P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _I64, _I64, _I64, _INT, _P],
    "daxq_linear_w8a8": [_INT, _INT, _INT, _P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _P, _I64, _I64, _I64, _I64, _INT, _P],
    "daxq_dynamic_linear": [_INT, _INT, _INT, _INT, _INT, _P, _I64, _P, _I64, _P, _I64, _P, _I64, _P, _P, _P, _I64, _I64, _I64, _I64,
                            _P, _I64, _INT, _P],
    "daxq_dynamic_linear_i8": [_P, _I64, _P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _I64, _I64, _I64, _P],
    "daxq_dynamic_linear_e4m3": [_P, _I64, _P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _I64, _I64, _I64, _P],
    "daxq_dynamic_linear_e5m2_e4m3": [_P, _I64, _P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _I64, _I64, _I64, _P],
}


class DaxqError(RuntimeError):
    """A daxq entry point returned a negative status."""


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise RuntimeError(
                        f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                        "(hipcc, gfx950). dax_amd has no other implementation to fall back to.")
                L = C.CDLL(LIB_PATH)
                for name, args in SIGNATURES.items():
                    fn = getattr(L, name)
                    fn.argtypes = args
                    fn.restype = (C.c_char_p if name == "daxq_last_error" else
                                  _I64 if name == "daxq_linear_splitk_workspace_bytes" else _INT)
                got = L.daxq_abi_version()
                if got != ABI_VERSION:
                    raise RuntimeError(f"libdaxq ABI {got} != expected {ABI_VERSION}; rebuild the library")
                _lib = L
    return _lib


def last_error() -> str:
    msg = lib().daxq_last_error()
    return msg.decode() if msg else ""


def check(status: int, what: str) -> None:
    if status != 0:
        raise DaxqError(f"{what} failed with status {status}: {last_error()}")


def device_info(device: int = 0) -> dict:
    cu, clk, lds = _INT(0), _INT(0), _INT(0)
    arch = C.create_string_buffer(64)
    st = lib().daxq_device_info(device, C.byref(cu), C.byref(clk), C.byref(lds), arch, 64)
    return {"status": st, "cu_count": cu.value, "clock_khz": clk.value, "lds_bytes": lds.value,
            "arch": arch.value.decode()}


def require_gfx950(device: int) -> None:
    """Raises unless `device` is a gfx950 (checked once per device); on the first check the library's kernels are
    prepared on that device (daxq_init), so that even the first op call may sit inside a stream capture."""
    if device in _checked_devices:
        return
    info = device_info(device)
    if info["status"] != 0:
        raise RuntimeError(f"daxq needs an MI355X (gfx950) device: {last_error()}")
    import torch

    with torch.cuda.device(device):
        check(lib().daxq_init(), "daxq_init")
    _checked_devices.add(device)


FMT = {"i8": 0, "e4m3": 1, "e5m2": 2}  # DAXQ_FMT_*
FLOAT_KIND = {"bf16": 0, "f16": 1, "f32": 2}  # DAXQ_BF16 / DAXQ_F16 / DAXQ_F32


# ---- test / comparison hook: which GEMM implementation the ops ask for (the `kernel` argument of daxq_linear_w8a8).
# Host-side only: the library itself keeps no selection, every call names its kernel.
_kernel_choice = 0
_tile_group = 0
_tile_order = 0
_tail = 0


def debug_select_gemm(v: int) -> None:
    """0 = the library's choice by shape; 2 / 5 / 8 / 11 / 14 = one implementation (include/daxq.h: the generic kernel on
    256x256 / 128x128 tiles, the tiled kernel on 256x256 / 128x128 / 256x128 tiles); 1000 + d = depth d of the tile-order groups
    (1000 = default); 2000 + o = tile order of the 256x256 kernels (2000 = by shape, 2001 = groups of tile rows,
    2002 = banded patches); 3000 + t = the last partial round of a 256x256 launch as 128x128 quadrants or 256x128 halves
    (3000 = by shape, 3001 = never, 3002 = whenever every such tile gets a CU)."""
    global _kernel_choice, _tile_group, _tile_order, _tail
    v = int(v)
    if 1000 <= v < 1064:
        _tile_group = v - 1000
    elif 2000 <= v < 2003:
        _tile_order = v - 2000
    elif 3000 <= v < 3003:
        _tail = v - 3000
    elif v in (0, 2, 5, 8, 11, 14):
        _kernel_choice = v
    else:
        raise DaxqError(f"unknown gemm kernel choice {v}")


def kernel_arg() -> int:
    return _kernel_choice | (_tile_group << 16) | (_tile_order << 24) | (_tail << 28)
