"""ctypes loader for the scalar C restatement (``codec_scalar.c``).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "_build" / "liboracle_scalar.so"
_lib = None


def build(force: bool = False) -> Path:
    """Compile the shared object with the committed Makefile."""
    if force or not _LIB_PATH.exists():
        subprocess.run(["make", "-C", str(_HERE)] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(str(build()))
        for name in ("lbo_quantize_f32", "lbo_dequantize_f32", "lbo_reduce_f32",
                     "lbo_ef_step_bf16", "lbo_ef_step_f32"):
            getattr(_lib, name).restype = None
    return _lib


def _ptr(array: np.ndarray | None):
    return None if array is None else array.ctypes.data_as(ctypes.c_void_p)


def quantize(x32: np.ndarray, group_size: int = 64):
    x32 = np.ascontiguousarray(x32, dtype=np.float32).reshape(-1)
    groups = -(-x32.size // group_size) if x32.size else 0
    codes = np.empty(groups * group_size, dtype=np.int8)
    scales = np.empty(groups, dtype=np.float32)
    lib().lbo_quantize_f32(_ptr(x32), ctypes.c_int64(x32.size), ctypes.c_int(group_size),
                           _ptr(codes), _ptr(scales))
    return codes, scales


def dequantize(codes: np.ndarray, scales: np.ndarray, numel: int, group_size: int = 64):
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    scales = np.ascontiguousarray(scales, dtype=np.float32)
    out = np.empty(numel, dtype=np.float32)
    lib().lbo_dequantize_f32(_ptr(codes), _ptr(scales), ctypes.c_int64(numel),
                             ctypes.c_int(group_size), _ptr(out))
    return out


def reduce_payloads(payloads, numel: int, group_size: int = 64, divisor: float = 1.0):
    world = len(payloads)
    codes = [np.ascontiguousarray(c, dtype=np.int8) for c, _ in payloads]
    scales = [np.ascontiguousarray(s, dtype=np.float32) for _, s in payloads]
    code_ptrs = (ctypes.c_void_p * world)(*[c.ctypes.data for c in codes])
    scale_ptrs = (ctypes.c_void_p * world)(*[s.ctypes.data for s in scales])
    out = np.empty(numel, dtype=np.float32)
    lib().lbo_reduce_f32(code_ptrs, scale_ptrs, ctypes.c_int(world), ctypes.c_int64(numel),
                         ctypes.c_int(group_size), ctypes.c_float(divisor), _ptr(out))
    return out


def ef_step_bf16(grad_bits: np.ndarray, residual32: np.ndarray | None, group_size: int = 64,
                 restored_bf16: bool = False):
    grad_bits = np.ascontiguousarray(grad_bits, dtype=np.uint16).reshape(-1)
    n = grad_bits.size
    if residual32 is not None:
        residual32 = np.ascontiguousarray(residual32, dtype=np.float32)
    groups = -(-n // group_size) if n else 0
    codes = np.empty(groups * group_size, dtype=np.int8)
    scales = np.empty(groups, dtype=np.float32)
    new_residual = np.empty(n, dtype=np.float32)
    restored = np.empty(n, dtype=np.uint16 if restored_bf16 else np.float32)
    lib().lbo_ef_step_bf16(_ptr(grad_bits), _ptr(residual32), ctypes.c_int64(n), ctypes.c_int(group_size),
                           _ptr(codes), _ptr(scales), _ptr(new_residual), _ptr(restored),
                           ctypes.c_int(1 if restored_bf16 else 0))
    return codes, scales, restored, new_residual


def ef_step_f32(grad32: np.ndarray, residual32: np.ndarray | None, group_size: int = 64):
    grad32 = np.ascontiguousarray(grad32, dtype=np.float32).reshape(-1)
    n = grad32.size
    if residual32 is not None:
        residual32 = np.ascontiguousarray(residual32, dtype=np.float32)
    groups = -(-n // group_size) if n else 0
    codes = np.empty(groups * group_size, dtype=np.int8)
    scales = np.empty(groups, dtype=np.float32)
    new_residual = np.empty(n, dtype=np.float32)
    restored = np.empty(n, dtype=np.float32)
    lib().lbo_ef_step_f32(_ptr(grad32), _ptr(residual32), ctypes.c_int64(n), ctypes.c_int(group_size),
                          _ptr(codes), _ptr(scales), _ptr(new_residual), _ptr(restored))
    return codes, scales, restored, new_residual
