"""CPU oracle (numpy) for the reference's CUDA wire format.  TEST INFRASTRUCTURE ONLY.

The reference's native extension (``ccdl_cuda_ops``) emits a payload that differs
from the portable codec's: the scale is the group's absolute maximum kept in the
tensor's own dtype, the encoder multiplies by ``127 / max(scale, 1e-6)``, codes are
byte-swapped inside 2-byte (fp16/bf16) or 4-byte (fp32) words, and the scales are
either interleaved after each group's codes (``compact``) or appended after all
codes.  This module restates that arithmetic and layout with numpy.  Only tests,
the smoke check and the benchmark's CPU-baseline leg may import it.

Reference lines each function follows (paths under the upstream repository):

* ``quantize``            ccdl_comm/csrc/quantization/quant_pack_kernel.cu:45-162
                          (fused compensate + absmax + encode + compact layout);
                          non-compact layout: quant_kernel_fp32.cuh:266-303,
                          quant_kernel.cuh:213-255
* ``split``               dequant_reduce_kernel.cu:27-69 (byte order and offsets as
                          the reader sees them)
* ``dequantize``          dequant_kernel_fp32.cuh:81-120, dequant_kernel.cuh:15-60
* ``reduce_payloads``     dequant_reduce_kernel.cu:71-134
* ``reduce_mean_error_feedback``
                          dequant_reduce_kernel.cu:150-221,355-430
* ``error_feedback_update``
                          dequant_reduce_kernel.cu:136-148,223-233

Pinning (tests/test_cuda_wire_oracle.py): writer and reader layouts are checked
against each other, codes against exact rational arithmetic on small inputs, the
numpy and scalar-C restatements against each other, invariants (extreme element
maps to +-127, stored scale equals the group maximum exactly, error bound), and
the round-trip error statistics the reference's benchmark reports record for fp16
and bf16 ``randn`` inputs.  The reference holds no golden payload bytes and no
CUDA device exists here, so agreement with an actual NVIDIA build is unpinned;
the accumulate in ``reduce_payloads`` in particular depends on whether nvcc fuses
``sum += code * scale`` into an FMA (its default), which is why it is a switch.

4-bit codes (``bit=4``; quant_pack_kernel.cu:103,120-130,145-158; inner.cuh:36-40,67-72): the multiplier is
``7 / max(scale, 1e-6)``, codes are clamped to +-7 and stored as two's-complement nibbles, four to a 16-bit
word or eight to a 32-bit word with the first element in the most significant nibble; decode multiplies the
sign-extended nibble by ``scale / 7``.  The reference has no fused reduce for them.

Arrays: fp32 -> ``float32``, fp16 -> ``float16``, bf16 -> ``uint16`` bit patterns.
"""
from __future__ import annotations

import numpy as np

from .codec_np import bf16_to_f32, f32_to_bf16

_ITEMSIZE = {"fp32": 4, "fp16": 2, "bf16": 2}
_F127 = np.float32(127.0)
_FLOOR = np.float32(1.0e-6)


def to_f32(values: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "bf16":
        return bf16_to_f32(values)
    return np.ascontiguousarray(values, dtype={"fp32": np.float32, "fp16": np.float16}[dtype]).astype(np.float32)


def from_f32(values: np.ndarray, dtype: str) -> np.ndarray:
    values = np.ascontiguousarray(values, dtype=np.float32)
    if dtype == "bf16":
        return f32_to_bf16(values)
    if dtype == "fp16":
        with np.errstate(over="ignore"):
            return values.astype(np.float16)
    return values


def _raw_bytes(values: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(values).view(np.uint8)


def num_groups(numel: int, group_size: int) -> int:
    return -(-numel // group_size) if numel else 0


def payload_nbytes(numel: int, group_size: int, dtype: str, bit: int = 8) -> int:
    """quant_pack_kernel.cu:247-249."""
    return num_groups(numel, group_size) * (group_size * bit // 8 + _ITEMSIZE[dtype])


def _levels(bit: int) -> np.float32:
    if bit not in (4, 8):
        raise ValueError(f"bit must be 4 or 8, got {bit}")
    return np.float32(127.0 if bit == 8 else 7.0)


def _pack_nibbles(codes: np.ndarray, word: int) -> np.ndarray:
    """int8 codes in [-7, 7] -> bytes: ``2*word`` consecutive codes fill one ``word``-byte little-endian unit with
    the first code in the most significant nibble (quant_pack_kernel.cu:123-129,149-157)."""
    nibbles = (codes.astype(np.int16) & 0xF).astype(np.uint8).reshape(-1, 2 * word)
    by_significance = (nibbles[:, 0::2] << 4) | nibbles[:, 1::2]        # most significant byte first
    return np.ascontiguousarray(by_significance[:, ::-1]).reshape(-1)


def _unpack_nibbles(code_bytes: np.ndarray, word: int) -> np.ndarray:
    by_significance = code_bytes.reshape(-1, word)[:, ::-1]
    nibbles = np.empty((by_significance.shape[0], 2 * word), dtype=np.uint8)
    nibbles[:, 0::2] = by_significance >> 4
    nibbles[:, 1::2] = by_significance & 0xF
    signed = nibbles.astype(np.int8)
    return np.where(signed >= 8, signed - 16, signed).astype(np.int8).reshape(-1)      # inner.cuh:36-40


def _swap_words(codes: np.ndarray, word: int) -> np.ndarray:
    """Byte order inside each ``word``-byte unit is reversed: the first code of a unit sits in its most
    significant byte (quant_pack_kernel.cu:111-118,131-143) and the unit is stored little-endian."""
    return np.ascontiguousarray(codes.reshape(-1, word)[:, ::-1]).reshape(-1)


def quantize(x: np.ndarray, dtype: str, group_size: int = 64, compact: bool = True,
             residual: np.ndarray | None = None, bit: int = 8) -> np.ndarray:
    levels = _levels(bit)
    xf = to_f32(x, dtype).reshape(-1)
    n = xf.size
    if residual is not None:
        with np.errstate(invalid="ignore", over="ignore"):
            xf = to_f32(from_f32(xf + to_f32(residual, dtype).reshape(-1), dtype), dtype)   # :87-91
    groups = num_groups(n, group_size)
    if groups == 0:
        return np.empty(0, dtype=np.uint8)
    padded = np.zeros(groups * group_size, dtype=np.float32)
    padded[:n] = xf
    rows = padded.reshape(groups, group_size)
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        absmax = np.fmax.reduce(np.abs(rows), axis=1, initial=np.float32(0.0)).astype(np.float32)   # fmaxf skips NaN
        stored = from_f32(absmax, dtype)                                                           # :101
        scale = np.fmax(to_f32(stored, dtype), _FLOOR)                                             # :102
        multiplier = (levels / scale).astype(np.float32)                                           # :103
        product = (rows * multiplier[:, None]).astype(np.float32)
        rounded = np.rint(product)
    rounded = np.where(np.isnan(rounded), np.float32(0.0), rounded)                                # __float2int_rn(NaN) = 0
    codes = np.clip(rounded, -levels, levels).astype(np.int8)
    if bit == 8:
        swapped = _swap_words(codes.view(np.uint8).reshape(-1), _ITEMSIZE[dtype]).reshape(groups, group_size)
    else:
        swapped = _pack_nibbles(codes.reshape(-1), _ITEMSIZE[dtype]).reshape(groups, group_size // 2)
    scale_bytes = _raw_bytes(stored).reshape(groups, _ITEMSIZE[dtype])
    if compact:
        return np.ascontiguousarray(np.concatenate([swapped, scale_bytes], axis=1)).reshape(-1)
    return np.concatenate([swapped.reshape(-1), scale_bytes.reshape(-1)])


def split(payload: np.ndarray, numel: int, dtype: str, group_size: int = 64, compact: bool = True, bit: int = 8):
    """Payload -> (int8 codes in element order [G*g], stored scales [G] in the payload dtype)."""
    _levels(bit)
    item = _ITEMSIZE[dtype]
    groups = num_groups(numel, group_size)
    per_group = group_size * bit // 8
    payload = np.ascontiguousarray(payload, dtype=np.uint8).reshape(-1)
    assert payload.size == groups * (per_group + item), (payload.size, groups, per_group, item)
    if compact:
        table = payload.reshape(groups, per_group + item)
        code_bytes = np.ascontiguousarray(table[:, :per_group]).reshape(-1)
        scale_bytes = np.ascontiguousarray(table[:, per_group:]).reshape(-1)
    else:
        code_bytes = payload[: groups * per_group]
        scale_bytes = np.ascontiguousarray(payload[groups * per_group:])
    codes = _swap_words(code_bytes, item).view(np.int8) if bit == 8 else _unpack_nibbles(code_bytes, item)
    view = {"fp32": np.float32, "fp16": np.float16, "bf16": np.uint16}[dtype]
    return codes, scale_bytes.view(view)


def _decode_f32(payload, numel, dtype, group_size, compact, bit=8):
    codes, stored = split(payload, numel, dtype, group_size, compact, bit)
    with np.errstate(invalid="ignore", over="ignore"):
        step = (to_f32(stored, dtype) / _levels(bit)).astype(np.float32)   # scale / 127 or scale / 7 (IEEE)
        values = codes.astype(np.float32).reshape(-1, group_size) * step[:, None]
    return values.astype(np.float32).reshape(-1)[:numel]


def _add_in_dtype(a: np.ndarray, b: np.ndarray, dtype: str) -> np.ndarray:
    """Correctly rounded a + b in ``dtype`` (one rounding), as a native half/bfloat16 add gives."""
    if dtype == "fp32":
        return (to_f32(a, dtype) + to_f32(b, dtype)).astype(np.float32)
    wide = to_f32(a, dtype).astype(np.float64) + to_f32(b, dtype).astype(np.float64)
    if dtype == "fp16":
        with np.errstate(over="ignore"):
            return wide.astype(np.float16)
    return _f64_to_bf16(wide)


def _f64_to_bf16(values: np.ndarray) -> np.ndarray:
    """float64 -> bf16 with a single rounding: round to odd into float32, then nearest-even to bf16."""
    with np.errstate(over="ignore", invalid="ignore"):
        near = values.astype(np.float32)
        err = values - near.astype(np.float64)
    bits = near.view(np.uint32).copy()
    inexact = (err != 0) & np.isfinite(near)
    even = (bits & np.uint32(1)) == 0
    # move an even, inexact result one step towards the true value so the low bit records the lost part
    towards_larger_magnitude = (err > 0) == (near > 0)
    step = np.where(towards_larger_magnitude, np.int64(1), np.int64(-1))
    adjust = inexact & even
    bits = np.where(adjust, (bits.astype(np.int64) + step).astype(np.uint32), bits)
    return f32_to_bf16(bits.view(np.float32))


def dequantize(payload: np.ndarray, numel: int, dtype: str, group_size: int = 64, compact: bool = True,
               reduce_op: str = "none", out: np.ndarray | None = None, bit: int = 8) -> np.ndarray:
    """Decode one payload into ``dtype``; SUM/MAX/MIN combine with the existing ``out`` in that dtype."""
    value = from_f32(_decode_f32(payload, numel, dtype, group_size, compact, bit), dtype)
    if reduce_op == "none":
        return value
    assert out is not None
    if reduce_op == "sum":
        return _add_in_dtype(out, value, dtype)
    old, new = to_f32(out, dtype), to_f32(value, dtype)
    if reduce_op == "max":      # (old > new) ? old : new
        pick_old = old > new
    elif reduce_op == "min":    # (old > new) ? new : old
        pick_old = ~(old > new)
    else:
        raise ValueError(reduce_op)
    return np.where(pick_old, np.asarray(out).reshape(-1), np.asarray(value).reshape(-1))


def fma_f32(a: np.ndarray, b: np.ndarray, c: np.ndarray) -> np.ndarray:
    """Correctly rounded float32 a*b+c for |a| < 2^8 integers: the product is exact in float64, the sum is
    formed with an error term and rounded to odd before the final float32 rounding."""
    prod = a.astype(np.float64) * b.astype(np.float64)
    c64 = c.astype(np.float64)
    with np.errstate(invalid="ignore", over="ignore"):
        s = prod + c64
        bb = s - prod
        err = (prod - (s - bb)) + (c64 - bb)
    bits = s.view(np.uint64).copy()
    inexact = np.isfinite(s) & (err != 0)
    even = (bits & np.uint64(1)) == 0
    towards_larger_magnitude = (err > 0) == (s > 0)
    step = np.where(towards_larger_magnitude, np.int64(1), np.int64(-1))
    bits = np.where(inexact & even, (bits.astype(np.int64) + step).astype(np.uint64), bits)
    with np.errstate(over="ignore", invalid="ignore"):
        return bits.view(np.float64).astype(np.float32)


def _accumulate(payloads, numel, dtype, group_size, compact, fused_multiply_add):
    groups = num_groups(numel, group_size)
    total = np.zeros(groups * group_size, dtype=np.float32)
    for payload in payloads:
        codes, stored = split(payload, numel, dtype, group_size, compact)
        with np.errstate(invalid="ignore", over="ignore"):
            step = np.repeat((to_f32(stored, dtype) / _F127).astype(np.float32), group_size)
            codes_f = codes.astype(np.float32)
            if fused_multiply_add:
                total = fma_f32(codes_f, step, total)
            else:
                total = (total + (codes_f * step).astype(np.float32)).astype(np.float32)
    return total[:numel]


def reduce_payloads(payloads, numel: int, dtype: str, group_size: int = 64, compact: bool = True,
                    inv_divisor: float = 1.0, fused_multiply_add: bool = True) -> np.ndarray:
    total = _accumulate(payloads, numel, dtype, group_size, compact, fused_multiply_add)
    with np.errstate(invalid="ignore", over="ignore"):
        return from_f32((total * np.float32(inv_divisor)).astype(np.float32), dtype)


def reduce_mean_error_feedback(payloads, prepared: np.ndarray, numel: int, dtype: str, group_size: int = 64,
                               compact: bool = True, divisor: int = 1, fused_multiply_add: bool = True):
    """-> (restored, residual); the residual subtracts the unrounded float32 mean (:181-183, :217-219)."""
    inv = np.float32(1.0) / np.float32(divisor)
    total = _accumulate(payloads, numel, dtype, group_size, compact, fused_multiply_add)
    with np.errstate(invalid="ignore", over="ignore"):
        mean = (total * inv).astype(np.float32)
        residual = (to_f32(prepared, dtype).reshape(-1) - mean).astype(np.float32)
    return from_f32(mean, dtype), from_f32(residual, dtype)


def error_feedback_update(prepared: np.ndarray, restored: np.ndarray, dtype: str) -> np.ndarray:
    with np.errstate(invalid="ignore", over="ignore"):
        return from_f32((to_f32(prepared, dtype) - to_f32(restored, dtype)).astype(np.float32), dtype)
