"""Payload sizing.

``estimate_quantized_size`` keeps the reference's signature and default arithmetic
(``ccdl_comm/quantization/sizing.py:52-91``): per group ``g*bit/8`` code bytes plus one scale stored
in the *source* dtype (2 bytes for fp16/bf16) plus top-k side data - the layout of the reference's
native CUDA buffers.  This package's kernels speak the portable codec's wire format instead, whose
scale is always fp32 (``ccdl_comm/quantization/torch_fallback.py:28-29``); pass
``wire_format="portable"`` (or call :func:`estimate_payload_size`) for that: 68 bytes per group of
64 for every source dtype.  For fp32 sources the two coincide.
"""
from __future__ import annotations

from dataclasses import dataclass

from lowbit_comm_amd.config import CompressionConfig

_ELEMENT_BYTES = {"fp16": 2, "bf16": 2, "fp32": 4}
# extra metadata bytes per group for top-k outliers, keyed by (is_fp32, topk)
_TOPK_BYTES = {(True, 0): 0, (True, 1): 8, (True, 2): 12, (False, 0): 0, (False, 1): 4, (False, 2): 6}
WIRE_FORMATS = ("native", "portable")


@dataclass(frozen=True)
class QuantizationSizeEstimate:
    """Storage footprint of one quantized tensor."""

    numel: int
    padded_numel: int
    padding_numel: int
    num_groups: int
    original_bytes: int
    quantized_bytes: int
    compression_ratio: float


def _element_bytes(dtype: str) -> int:
    if dtype not in _ELEMENT_BYTES:
        raise ValueError(f"Unsupported dtype={dtype!r}; expected one of {sorted(_ELEMENT_BYTES)}")
    return _ELEMENT_BYTES[dtype]


def estimate_quantized_size(numel: int, *, dtype: str, config: CompressionConfig,
                            wire_format: str = "native") -> QuantizationSizeEstimate:
    """Size of the quantized buffer for ``numel`` elements of ``dtype`` under ``config``."""
    if numel < 0:
        raise ValueError("numel must be non-negative")
    if wire_format not in WIRE_FORMATS:
        raise ValueError(f"Unsupported wire_format={wire_format!r}; expected one of {list(WIRE_FORMATS)}")
    source_bytes = _element_bytes(dtype)
    g = config.group_size
    groups = -(-numel // g) if numel else 0
    scale_bytes = 4 if wire_format == "portable" else source_bytes
    per_group = g * config.bit // 8 + scale_bytes + _TOPK_BYTES[(dtype == "fp32", config.topk)]
    quantized = groups * per_group
    original = numel * source_bytes
    return QuantizationSizeEstimate(
        numel=numel,
        padded_numel=groups * g,
        padding_numel=groups * g - numel,
        num_groups=groups,
        original_bytes=original,
        quantized_bytes=quantized,
        compression_ratio=original / quantized if quantized else 0.0,
    )


def estimate_payload_size(numel: int, *, dtype: str, config: CompressionConfig) -> QuantizationSizeEstimate:
    """Size of a packed ``uint8[codes || fp32 scales]`` payload as this package's kernels write it."""
    return estimate_quantized_size(numel, dtype=dtype, config=config, wire_format="portable")
