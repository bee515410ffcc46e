"""ctypes loader for the scalar C restatement of the general CUDA kernels (``cuda_wire_general_scalar.c``).
TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes

import numpy as np

from . import scalar as _scalar
from .cuda_wire_general_np import QUANT_TYPES, payload_nbytes

_DTYPE = {"fp32": 0, "fp16": 1, "bf16": 2}
_NUMPY = {"fp32": np.float32, "fp16": np.float16, "bf16": np.uint16}
_OPS = {"none": 0, "sum": 1, "max": 2, "min": 3}


def _lib() -> ctypes.CDLL:
    lib = _scalar.lib()
    for name in ("lbg_quantize", "lbg_dequantize", "lbg_philox_block", "lbg_curand_draws"):
        getattr(lib, name).restype = None
    return lib


def _ptr(array):
    return array.ctypes.data_as(ctypes.c_void_p)


def philox_block(counter, key) -> np.ndarray:
    counter = np.ascontiguousarray(counter, dtype=np.uint32)
    key = np.ascontiguousarray(key, dtype=np.uint32)
    out = np.zeros(4, dtype=np.uint32)
    _lib().lbg_philox_block(_ptr(counter), _ptr(key), _ptr(out))
    return out


def curand_draws(seed: int, subsequence: int, offset: int, count: int) -> np.ndarray:
    out = np.zeros(count, dtype=np.uint32)
    _lib().lbg_curand_draws(ctypes.c_uint64(seed), ctypes.c_uint64(subsequence), ctypes.c_uint64(offset),
                            ctypes.c_int(count), _ptr(out))
    return out


def quantize(x, dtype: str, group_size: int = 64, bit: int = 8, quant_type: str = "linear", topk: int = 0,
             stochastic: tuple[int, int] | None = None, compact: bool = False) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=_NUMPY[dtype]).reshape(-1)
    assert x.size % group_size == 0
    payload = np.zeros(payload_nbytes(x.size, group_size, dtype, bit, topk), dtype=np.uint8)
    seed, offset = stochastic if stochastic is not None else (0, 0)
    _lib().lbg_quantize(_ptr(x), ctypes.c_int(_DTYPE[dtype]), ctypes.c_int64(x.size), ctypes.c_int(group_size),
                        ctypes.c_int(bit), ctypes.c_int(QUANT_TYPES.index(quant_type)), ctypes.c_int(topk),
                        ctypes.c_int(int(stochastic is not None)), ctypes.c_uint64(seed), ctypes.c_uint64(offset),
                        ctypes.c_int(int(compact)), _ptr(payload))
    return payload


def dequantize(payload, numel: int, dtype: str, group_size: int = 64, bit: int = 8, quant_type: str = "linear",
               topk: int = 0, compact: bool = False, reduce_op: str = "none", out=None) -> np.ndarray:
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    if out is None:
        result = np.zeros(numel, dtype=_NUMPY[dtype])
    else:
        result = np.ascontiguousarray(out, dtype=_NUMPY[dtype]).reshape(-1).copy()
    _lib().lbg_dequantize(_ptr(payload), ctypes.c_int64(numel), ctypes.c_int(group_size), ctypes.c_int(bit),
                          ctypes.c_int(QUANT_TYPES.index(quant_type)), ctypes.c_int(topk), ctypes.c_int(int(compact)),
                          ctypes.c_int(_DTYPE[dtype]), ctypes.c_int(_OPS[reduce_op]), _ptr(result))
    return result
