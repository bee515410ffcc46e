"""ctypes binding of ``liblbc_hip.so`` (the C ABI declared in ``include/lbc.h``).

The library is built in-tree by ``lowbit_comm_amd/csrc/Makefile``.  Loading never falls back to
anything else: if the shared object is missing or a symbol is absent, :func:`load_library` raises.
"""
from __future__ import annotations

import ctypes
from pathlib import Path

from lowbit_comm_amd.exceptions import CCDLUnavailableError

LIBRARY_PATH = Path(__file__).resolve().parent.parent / "liblbc_hip.so"
ABI_VERSION = 8

LBC_OK = 0
LBC_UNSUPPORTED = 1

_c_ptr = ctypes.c_void_p
_c_i64 = ctypes.c_int64
_c_int = ctypes.c_int

# symbol -> (restype, argtypes); one entry per declaration in include/lbc.h
SIGNATURES = {
    "lbc_abi_version": (_c_int, []),
    "lbc_last_error": (ctypes.c_char_p, []),
    "lbc_quant_pack": (_c_int, [_c_ptr, _c_int, _c_ptr, _c_int, _c_i64, _c_int, _c_ptr, _c_ptr,
                                _c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr]),
    "lbc_quant_pack_chunks": (_c_int, [_c_ptr, _c_int, _c_ptr, _c_int, _c_i64, _c_int, _c_int, _c_ptr, _c_i64,
                                       _c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr]),
    "lbc_dequant": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_ptr]),
    "lbc_dequant_chunks": (_c_int, [_c_ptr, _c_i64, _c_int, _c_i64, _c_i64, _c_int, _c_ptr, _c_int, _c_int, _c_ptr]),
    "lbc_dequant_reduce": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_int, ctypes.c_float, _c_ptr, _c_int,
                                    _c_ptr, _c_ptr, _c_int, _c_ptr]),
    "lbc_quant_pack_chunks_and_dequant_reduce": (_c_int, [
        _c_ptr, _c_int, _c_ptr, _c_int, _c_i64, _c_int, _c_int, _c_ptr, _c_i64, _c_ptr, _c_int,
        _c_ptr, _c_ptr, _c_int, _c_i64, ctypes.c_float, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr]),
    "lbc_dequant_reduce_quant": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_int, ctypes.c_float, _c_int, _c_ptr,
                                          _c_ptr, _c_int, _c_ptr]),
    "lbc_bucket_pipeline_step": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr]),
    "lbc_ring_step": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int, ctypes.c_float, _c_ptr, _c_ptr,
                               _c_int, _c_ptr]),
    "lbc_ef_update": (_c_int, [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_int, _c_i64, _c_int, _c_ptr]),
    "lbc_wire_payload_nbytes": (_c_i64, [_c_i64, _c_int, _c_int, _c_int]),
    "lbc_wire_quant_pack": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_ptr]),
    "lbc_wire_quant_pack_chunks": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_ptr,
                                            _c_i64, _c_int, _c_ptr]),
    "lbc_wire_ring_step": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_i64, _c_int, _c_int, _c_int, ctypes.c_float, _c_ptr, _c_int, _c_ptr]),
    "lbc_wire_dequant": (_c_int, [_c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_ptr]),
    "lbc_wire_dequant_chunks": (_c_int, [_c_ptr, _c_i64, _c_int, _c_i64, _c_i64, _c_int, _c_int, _c_int, _c_ptr,
                                         _c_int, _c_int, _c_int, _c_ptr]),
    "lbc_wire_dequant_reduce": (_c_int, [_c_ptr, _c_int, _c_i64, _c_int, _c_int, ctypes.c_float, _c_int, _c_ptr,
                                         _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr]),
    "lbc_wire_general_payload_nbytes": (_c_i64, [_c_i64, _c_int, _c_int, _c_int, _c_int]),
    "lbc_wire_quant_general": (_c_int, [_c_ptr, _c_int, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, ctypes.c_uint64,
                                        ctypes.c_uint64, _c_int, _c_ptr, _c_ptr]),
    "lbc_wire_dequant_general": (_c_int, [_c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_int,
                                          _c_int, _c_ptr]),
}



class QuantChunksStage(ctypes.Structure):
    """``lbc_quant_chunks_stage`` of include/lbc.h."""

    _fields_ = [("x", _c_ptr), ("residual", _c_ptr), ("payloads", _c_ptr), ("new_residual", _c_ptr),
                ("numel", _c_i64), ("payload_stride", _c_i64),
                ("x_dtype", _c_int), ("residual_dtype", _c_int), ("new_residual_dtype", _c_int), ("world", _c_int)]


class ReduceQuantStage(ctypes.Structure):
    """``lbc_reduce_quant_stage`` of include/lbc.h."""

    _fields_ = [("codes", _c_ptr), ("scales", _c_ptr), ("out_codes", _c_ptr), ("out_scales", _c_ptr),
                ("numel", _c_i64), ("divisor", ctypes.c_float), ("world", _c_int), ("mid_dtype", _c_int)]


class DequantChunksStage(ctypes.Structure):
    """``lbc_dequant_chunks_stage`` of include/lbc.h."""

    _fields_ = [("payloads", _c_ptr), ("out", _c_ptr), ("payload_stride", _c_i64), ("shard_numel", _c_i64),
                ("total_numel", _c_i64), ("world", _c_int), ("out_dtype", _c_int)]


_library: ctypes.CDLL | None = None


def load_library(path: str | Path | None = None) -> ctypes.CDLL:
    """Load the shared object once and type every entry point."""
    global _library
    if _library is not None and path is None:
        return _library
    target = Path(path) if path is not None else LIBRARY_PATH
    if not target.exists():
        raise CCDLUnavailableError(
            f"{target.name} is not built (run `make -C lowbit_comm_amd/csrc` or __graft_entry__.build())")
    try:
        lib = ctypes.CDLL(str(target))
    except OSError as exc:
        raise CCDLUnavailableError(f"cannot load {target}: {exc}") from exc
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise CCDLUnavailableError(f"{target.name} missing required symbol: {name}") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    version = lib.lbc_abi_version()
    if version != ABI_VERSION:
        raise CCDLUnavailableError(f"{target.name} has ABI version {version}, expected {ABI_VERSION}")
    if path is None:
        _library = lib
    return lib


def last_error(lib: ctypes.CDLL) -> str:
    raw = lib.lbc_last_error()
    return raw.decode("utf-8", "replace") if raw else ""
