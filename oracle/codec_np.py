"""CPU oracle (numpy) for the INT8 group codec.  TEST INFRASTRUCTURE ONLY.

This module restates, with numpy float32 arithmetic, the algorithm of the
reference's portable codec.  Only tests, the smoke check and the CPU-baseline
leg of the benchmark may import it; the product never routes through it.

Reference lines each function follows (paths under the upstream repository):

* ``quantize``          ccdl_comm/quantization/torch_fallback.py:24-36,56-61
* ``dequantize``        ccdl_comm/quantization/torch_fallback.py:48-53
* ``reduce_payloads``   ccdl_comm/communication/gather_reduce.py:27-45
* ``pack`` / ``unpack`` ccdl_comm/communication/payload_packing.py:63-75,190-198
* ``ef_compensate`` / ``ef_residual``
                        ccdl_comm/quantization/error_feedback.py:27-41
* ``ef_round_trip``     ccdl_comm/communication/ddp.py:69-97 (all_reduce=None)
* ``chunk_plan``        ccdl_comm/cuda/transports/compressed_reduce_scatter.py:72-94
* ``reduce_scatter_all_gather_plan``
                        ccdl_comm/communication/reduce_scatter_transport.py:252-276,688-696
                        and ccdl_comm/communication/topology_transport.py:866-894

Pinning (tests/test_oracle_pins.py): every function is checked against the
literal vectors the reference's own tests hold (packer bytes, error-feedback
cycles), against an independent scalar C restatement and a torch-op
restatement, against brute-force Python-float arithmetic on tiny inputs, and
against invariants a wrong sign / index / dropped clamp would break.

Numeric policy for values the reference leaves undefined (an int8 cast of a
NaN): a non-finite quotient encodes as code 0 when NaN and saturates to +-127
when infinite; the scale keeps the NaN/Inf bits.

16-bit floats: fp16 uses numpy's float16; bf16 has no numpy dtype, so bf16
arrays are carried as ``uint16`` bit patterns (see ``bf16_to_f32`` and
``f32_to_bf16``).
"""
from __future__ import annotations

import numpy as np

F32_EPS = np.float32(2.0 ** -23)  # torch.finfo(torch.float32).eps
_F127 = np.float32(127.0)


# --------------------------------------------------------------------------- #
# dtype plumbing
# --------------------------------------------------------------------------- #
def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    """Widen bf16 bit patterns (uint16) to float32; exact."""
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16(values: np.ndarray) -> np.ndarray:
    """Round float32 to bf16 bit patterns, nearest-even, NaN kept quiet."""
    u = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = (u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    is_nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    quiet = (u >> np.uint32(16)) | np.uint32(0x0040)
    return np.where(is_nan, quiet, rounded).astype(np.uint16)


def widen(values: np.ndarray, dtype: str) -> np.ndarray:
    """Return the float32 view of an fp32 / fp16 / bf16(bits) array."""
    if dtype == "fp32":
        return np.ascontiguousarray(values, dtype=np.float32)
    if dtype == "fp16":
        return np.ascontiguousarray(values, dtype=np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_to_f32(values)
    raise ValueError(f"unsupported dtype {dtype!r}")


def narrow(values: np.ndarray, dtype: str) -> np.ndarray:
    """Round float32 to ``dtype`` (bf16 comes back as uint16 bits)."""
    values = np.ascontiguousarray(values, dtype=np.float32)
    if dtype == "fp32":
        return values
    if dtype == "fp16":
        return values.astype(np.float16)
    if dtype == "bf16":
        return f32_to_bf16(values)
    raise ValueError(f"unsupported dtype {dtype!r}")


def _round_through(values: np.ndarray, dtype: str) -> np.ndarray:
    """float32 -> dtype -> float32 (the value an array of ``dtype`` holds)."""
    return widen(narrow(values, dtype), dtype)


# --------------------------------------------------------------------------- #
# quantize / dequantize
# --------------------------------------------------------------------------- #
def quantize(x32: np.ndarray, group_size: int = 64):
    """Group-wise linear INT8 quantization of a flat float32 array.

    Returns ``(codes int8[G*g], scales float32[G])``; the tail group is zero
    padded, so padding codes are 0.
    """
    flat = np.ascontiguousarray(x32, dtype=np.float32).reshape(-1)
    n = flat.size
    groups_n = -(-n // group_size) if n else 0
    padded = np.zeros(groups_n * group_size, dtype=np.float32)
    padded[:n] = flat
    groups = padded.reshape(groups_n, group_size)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        absmax = np.max(np.abs(groups), axis=1) if groups_n else np.zeros(0, np.float32)
        scales = np.maximum(absmax / _F127, F32_EPS).astype(np.float32)
        quotient = groups / scales[:, None]
        rounded = np.rint(quotient)
        clipped = np.clip(rounded, np.float32(-127.0), np.float32(127.0))
        clipped = np.where(np.isnan(clipped), np.float32(0.0), clipped)
    return clipped.astype(np.int8).reshape(-1), scales


def dequantize(codes: np.ndarray, scales: np.ndarray, numel: int, group_size: int = 64,
               dtype: str = "fp32") -> np.ndarray:
    """``float(code) * scale`` (one rounding), trimmed to ``numel``, cast to ``dtype``."""
    groups = np.ascontiguousarray(codes, dtype=np.int8).reshape(-1, group_size).astype(np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        restored = groups * np.ascontiguousarray(scales, dtype=np.float32)[:, None]
    return narrow(restored.reshape(-1)[:numel], dtype)


def reduce_payloads(payloads, numel: int, group_size: int = 64, dtype: str = "fp32",
                    reduce: str = "sum") -> np.ndarray:
    """Decode every payload to ``dtype`` and left-fold them in list order.

    Each partial sum is rounded to ``dtype`` (a bf16 bucket adds in bf16);
    ``mean`` divides by the payload count with a true division in ``dtype``.
    """
    if not payloads:
        raise ValueError("cannot reduce an empty payload list")
    if reduce not in ("sum", "mean"):
        raise ValueError(f"unsupported gather-reduce mode: {reduce}")
    decoded = [widen(dequantize(c, s, numel, group_size, dtype), dtype) for c, s in payloads]
    total = decoded[0]
    with np.errstate(invalid="ignore", over="ignore"):
        for term in decoded[1:]:
            total = _round_through(total + term, dtype)
        if reduce == "mean":
            total = _round_through(total / np.float32(len(payloads)), dtype)
    return narrow(total, dtype)


# --------------------------------------------------------------------------- #
# wire format
# --------------------------------------------------------------------------- #
def pack(codes: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """``uint8[codes || scales]``: int8 two's complement, then fp32 little-endian."""
    code_bytes = np.ascontiguousarray(codes, dtype=np.int8).view(np.uint8).reshape(-1)
    scale_bytes = np.ascontiguousarray(scales, dtype="<f4").view(np.uint8).reshape(-1)
    return np.concatenate([code_bytes, scale_bytes])


def unpack(packed: np.ndarray, groups_n: int, group_size: int = 64):
    """Inverse of :func:`pack` for a payload of ``groups_n`` groups."""
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    code_bytes = groups_n * group_size
    if packed.size != code_bytes + 4 * groups_n:
        raise ValueError("packed payload has the wrong byte count")
    codes = packed[:code_bytes].view(np.int8)
    scales = packed[code_bytes:].copy().view("<f4").astype(np.float32)
    return codes, scales


# --------------------------------------------------------------------------- #
# error feedback
# --------------------------------------------------------------------------- #
def ef_compensate(grad: np.ndarray, grad_dtype: str, residual32: np.ndarray | None) -> np.ndarray:
    """``grad + residual`` with torch promotion (16-bit + fp32 -> fp32)."""
    g32 = widen(grad, grad_dtype)
    if residual32 is None:
        return g32
    return g32 + np.ascontiguousarray(residual32, dtype=np.float32)


def ef_residual(prepared32: np.ndarray, restored: np.ndarray, restored_dtype: str) -> np.ndarray:
    """``prepared - restored`` in fp32."""
    with np.errstate(invalid="ignore", over="ignore"):
        return np.ascontiguousarray(prepared32, dtype=np.float32) - widen(restored, restored_dtype)


def ef_round_trip(grad: np.ndarray, grad_dtype: str, residual32: np.ndarray | None,
                  group_size: int = 64, restored_dtype: str = "fp32"):
    """One local bucket step: p = g + r, q = quant(p), restored = dequant(q), r' = p - restored.

    Returns ``(codes, scales, restored[restored_dtype], new_residual float32)``.
    """
    prepared = ef_compensate(grad, grad_dtype, residual32)
    codes, scales = quantize(prepared, group_size)
    restored = dequantize(codes, scales, prepared.size, group_size, restored_dtype)
    return codes, scales, restored, ef_residual(prepared, restored, restored_dtype)


# --------------------------------------------------------------------------- #
# reduce-scatter + all-gather plan on one device
# --------------------------------------------------------------------------- #
def chunk_plan(original_numel: int, world_size: int):
    """Equal contiguous destination chunks: ``(shard_numel, padded_numel, [(start, stop)])``."""
    if original_numel < 0:
        raise ValueError("original_numel must be >= 0")
    if world_size <= 0:
        raise ValueError("world_size must be > 0")
    shard = (original_numel + world_size - 1) // world_size
    return shard, shard * world_size, [(r * shard, (r + 1) * shard) for r in range(world_size)]


def quantize_chunks(x32: np.ndarray, world_size: int, group_size: int = 64):
    """Zero-pad to ``W * shard`` and quantize each destination chunk on its own."""
    flat = np.ascontiguousarray(x32, dtype=np.float32).reshape(-1)
    shard, padded_numel, ranges = chunk_plan(flat.size, world_size)
    padded = np.zeros(padded_numel, dtype=np.float32)
    padded[: flat.size] = flat
    return [quantize(padded[a:b], group_size) for a, b in ranges]


def reduce_scatter_all_gather_plan(peer_buckets32, group_size: int = 64, reduce: str = "sum"):
    """Full compressed plan with every rank simulated on the host.

    ``peer_buckets32``: W float32 buckets of equal length (one per rank).
    Rank ``d`` reduces chunk ``d`` of all W peers (rank order), requantizes its
    shard, and every rank decodes the W requantized shards back into a bucket.
    Returns ``(shards float32 [W][shard_numel], restored float32 [n])``.
    """
    world = len(peer_buckets32)
    n = int(np.asarray(peer_buckets32[0]).size)
    shard, _padded, _ranges = chunk_plan(n, world)
    per_peer = [quantize_chunks(b, world, group_size) for b in peer_buckets32]
    shards = []
    for dest in range(world):
        received = [per_peer[src][dest] for src in range(world)]
        shards.append(reduce_payloads(received, shard, group_size, "fp32", reduce))
    gathered = [quantize(s, group_size) for s in shards]
    decoded = [dequantize(c, s, shard, group_size, "fp32") for c, s in gathered]
    restored = np.concatenate(decoded)[:n] if decoded else np.zeros(0, np.float32)
    return shards, restored
