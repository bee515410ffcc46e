"""ctypes loader for the scalar C restatement of the CUDA wire format (``cuda_wire_scalar.c``).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes

import numpy as np

from . import scalar as _scalar
from .cuda_wire_np import payload_nbytes

_DTYPE = {"fp32": 0, "fp16": 1, "bf16": 2}
_NUMPY = {"fp32": np.float32, "fp16": np.float16, "bf16": np.uint16}
_OPS = {"none": 0, "sum": 1, "max": 2, "min": 3}


def _lib() -> ctypes.CDLL:
    lib = _scalar.lib()
    for name in ("lbw_quantize", "lbw_dequantize", "lbw_reduce"):
        getattr(lib, name).restype = None
    return lib


def _ptr(array):
    return None if array is None else array.ctypes.data_as(ctypes.c_void_p)


def _typed(values, dtype):
    return np.ascontiguousarray(values, dtype=_NUMPY[dtype]).reshape(-1)


def quantize(x, dtype: str, group_size: int = 64, compact: bool = True, residual=None, bit: int = 8) -> np.ndarray:
    x = _typed(x, dtype)
    residual = None if residual is None else _typed(residual, dtype)
    payload = np.zeros(payload_nbytes(x.size, group_size, dtype, bit), dtype=np.uint8)
    _lib().lbw_quantize(_ptr(x), _ptr(residual), ctypes.c_int(_DTYPE[dtype]), ctypes.c_int64(x.size),
                        ctypes.c_int(group_size), ctypes.c_int(int(compact)), ctypes.c_int(bit), _ptr(payload))
    return payload


def dequantize(payload, numel: int, dtype: str, group_size: int = 64, compact: bool = True,
               reduce_op: str = "none", out=None, bit: int = 8) -> np.ndarray:
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    result = np.zeros(numel, dtype=_NUMPY[dtype]) if out is None else _typed(out, dtype).copy()
    _lib().lbw_dequantize(_ptr(payload), ctypes.c_int64(numel), ctypes.c_int(group_size), ctypes.c_int(int(compact)),
                          ctypes.c_int(_DTYPE[dtype]), ctypes.c_int(_OPS[reduce_op]), ctypes.c_int(bit), _ptr(result))
    return result


def reduce_payloads(payloads, numel: int, dtype: str, group_size: int = 64, compact: bool = True,
                    inv_divisor: float = 1.0, fused_multiply_add: bool = True, prepared=None):
    """-> out, or (out, residual) when ``prepared`` is given."""
    held = [np.ascontiguousarray(p, dtype=np.uint8) for p in payloads]
    pointers = (ctypes.c_void_p * len(held))(*[p.ctypes.data for p in held])
    out = np.zeros(numel, dtype=_NUMPY[dtype])
    prepared = None if prepared is None else _typed(prepared, dtype)
    residual = None if prepared is None else np.zeros(numel, dtype=_NUMPY[dtype])
    _lib().lbw_reduce(pointers, ctypes.c_int(len(held)), ctypes.c_int64(numel), ctypes.c_int(group_size),
                      ctypes.c_int(int(compact)), ctypes.c_int(_DTYPE[dtype]), ctypes.c_float(inv_divisor),
                      ctypes.c_int(int(fused_multiply_add)), _ptr(prepared), _ptr(out), _ptr(residual))
    return out if prepared is None else (out, residual)
