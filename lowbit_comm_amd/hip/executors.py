"""Executor for payloads that are already gathered in device memory - the reference's own single-GPU
entry point ``run_precollected_payloads(payloads, prepared, output, residual)``
(``ccdl_comm/cuda/executors.py:66-119`` over ``ccdl_comm/cuda/compiler.py:700-866``).

It reduces the rank payloads into the caller-owned ``output`` with a mean, and writes
``residual = prepared - output``, in one fused launch; when the fused call declines (more than 8
payloads, unsupported policy, layout the kernel rejects) it runs the chain decode-reduce ->
divide -> residual update and records why.
"""
from __future__ import annotations

from dataclasses import dataclass
from math import prod
from typing import Any

from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.execution_info import ExecutionCounters, ExecutionInfo
from lowbit_comm_amd.quantization.codec import (
    dequantize_reduce_tensors,
    inplace_dequantize_reduce_mean_update_error_feedback,
    update_error_feedback_residual,
)
from lowbit_comm_amd.quantization.sizing import estimate_quantized_size

FUSED_FAST_PATH = "hip_fused_dequant_reduce_mean_ef"
MAX_FUSED_PAYLOADS = 8


@dataclass(frozen=True)
class PrecollectedPayloadExecution:
    """Outcome of one precollected reduction."""

    output: object
    fused: bool
    fallback_reason: str | None = None

    def __post_init__(self) -> None:
        if self.fused and self.fallback_reason is not None:
            raise ValueError("fused execution must not provide a fallback reason")
        if not self.fused and not self.fallback_reason:
            raise ValueError("fallback execution requires a fallback reason")


def fused_dequant_fallback_reason(config: CompressionConfig) -> str | None:
    """Why the fused kernel cannot serve ``config`` (``None`` when it can)."""
    if config.group_size not in (16, 32, 64):
        return f"fused dequant requires group_size 16, 32 or 64; received {config.group_size}"
    if config.topk != 0:
        return f"fused dequant requires topk=0; received {config.topk}"
    if config.bit != 8:
        return f"fused dequant requires bit=8; received {config.bit}"
    if config.quant_type != "linear":
        return f"fused dequant requires quant_type='linear'; received {config.quant_type!r}"
    return None


def _buffer_of(payload: object) -> object:
    return payload.buffer if hasattr(payload, "buffer") else payload


def validate_precollected_payloads(buffers: list, *, expected_bytes: int, output: object) -> None:
    """Each payload must be ``uint8``, of exactly ``expected_bytes`` bytes, on ``output``'s device."""
    device = getattr(output, "device", None)
    for i, buffer in enumerate(buffers):
        numel, dtype, where = getattr(buffer, "numel", None), getattr(buffer, "dtype", None), getattr(buffer, "device", None)
        if not callable(numel) or dtype is None or where is None:
            continue
        if int(numel()) != expected_bytes:
            raise ValueError(f"payload[{i}] must contain {expected_bytes} bytes; received {int(numel())}")
        if str(dtype).removeprefix("torch.") != "uint8":
            raise TypeError(f"payload[{i}] must have dtype uint8; received {dtype}")
        if device is not None and where != device:
            raise ValueError(f"payload[{i}] must be on output device {device}; received {where}")


class PrecollectedPayloadExecutor:
    """Pre-bound ``mean``-reduction of gathered payloads with fused error-feedback update."""

    def __init__(self, config: CompressionConfig, *, shape: tuple[int, ...], dtype: str,
                 extension_status: Any | None = None, wire_format: str = "portable") -> None:
        self.config = config
        self.shape = tuple(shape)
        self.dtype = dtype
        self.extension_status = extension_status
        numel = prod(self.shape)
        estimate = estimate_quantized_size(numel, dtype=dtype, config=config, wire_format=wire_format)
        self.expected_payload_bytes = estimate.quantized_bytes
        self._static_reason = fused_dequant_fallback_reason(config)
        self.execution_info = ExecutionInfo.for_fused_path(
            strategy="all_gather", fast_path=FUSED_FAST_PATH, stage="dequant_reduce_mean_ef",
            original_bytes=estimate.original_bytes, compressed_bytes=estimate.quantized_bytes)
        self.last_execution_info = self.execution_info
        self.execution_counters = ExecutionCounters()

    def _run(self, payloads: object, prepared: object, output: object, residual: object) -> PrecollectedPayloadExecution:
        buffers = [_buffer_of(p) for p in payloads]
        if not buffers:
            raise ValueError("payloads must not be empty")
        validate_precollected_payloads(buffers, expected_bytes=self.expected_payload_bytes, output=output)
        runtime_reason = None
        if len(buffers) > MAX_FUSED_PAYLOADS:
            runtime_reason = f"fused dequant supports at most {MAX_FUSED_PAYLOADS} payloads; received {len(buffers)}"
        if self._static_reason is None and runtime_reason is None:
            if inplace_dequantize_reduce_mean_update_error_feedback(
                    buffers, prepared, output, residual, self.config, extension_status=self.extension_status,
                    reduce="mean"):
                return PrecollectedPayloadExecution(output=output, fused=True)
        restored = dequantize_reduce_tensors(buffers, self.shape, self.config, dtype=self.dtype,
                                             extension_status=self.extension_status, output=output, reduce="sum")
        if len(buffers) != 1:
            if getattr(restored, "is_cuda", False):
                from lowbit_comm_amd.hip.ops import true_divide_

                true_divide_(restored, len(buffers))
            else:
                restored.div_(len(buffers))
        update_error_feedback_residual(prepared, restored, residual, extension_status=self.extension_status)
        reason = self._static_reason or runtime_reason or "native fused dequant-reduce rejected runtime tensor layout"
        return PrecollectedPayloadExecution(output=output, fused=False, fallback_reason=reason)

    def run_precollected_payloads(self, payloads: object, prepared: object, output: object, residual: object) -> object:
        """Reduce into ``output`` (mean over payloads) and refresh ``residual``; returns ``output``."""
        self.execution_counters._record_run()
        try:
            execution = self._run(payloads, prepared, output, residual)
        except BaseException:
            self.execution_counters._record_failed()
            raise
        if execution.fused:
            self.last_execution_info = self.execution_info
        else:
            self.last_execution_info = self.execution_info.with_fallback(execution.fallback_reason)
        self.execution_counters._record_completed()
        return execution.output
