"""Synchronous compressed bucket processing (``ccdl_comm/communication/ddp.py:33-97``).

``process`` runs ``compensate -> quantize -> [all_reduce] -> dequantize -> residual update`` for one
DDP bucket and never touches ``torch.distributed`` itself.  ``from_hip_codec`` binds the GPU codec;
with ``fused=True`` and no collective the whole local round trip is a single kernel.
"""
from __future__ import annotations

from collections.abc import Callable, Hashable
from dataclasses import dataclass, field
from typing import Any

from lowbit_comm_amd.communication.collectives import CompressedAllReduce, CompressedPayload
from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.quantization.error_feedback import ErrorFeedbackState


def bucket_key(bucket: Any) -> Hashable:
    index = getattr(bucket, "index", None)
    return index() if callable(index) else id(bucket)


def bucket_tensor(bucket: Any) -> Any:
    buffer = getattr(bucket, "buffer", None)
    if not callable(buffer):
        raise TypeError("DDP bucket object must provide a callable buffer() method")
    return buffer()


@dataclass
class DDPBucketProcessor:
    config: CompressionConfig
    quantize: Callable[[Any, CompressionConfig], Any]
    dequantize: Callable[[Any, tuple[int, ...], CompressionConfig, str], Any]
    all_reduce: Callable[[CompressedPayload, str], CompressedPayload] | None = None
    error_feedback: ErrorFeedbackState = field(default_factory=ErrorFeedbackState)
    fused_codec: Any | None = None  # a FusedErrorFeedbackCodec, used when there is no collective

    @classmethod
    def from_cuda_codec(cls, config: CompressionConfig, *, extension_status: Any | None = None,
                        error_feedback: ErrorFeedbackState | None = None) -> "DDPBucketProcessor":
        """Bind the codec facade (flat ``uint8`` buffers) - the reference's constructor name."""
        from lowbit_comm_amd.quantization.codec import dequantize_tensor, quantize_tensor

        def quantize(tensor: Any, active: CompressionConfig) -> Any:
            return quantize_tensor(tensor, active, extension_status=extension_status)

        def dequantize(payload: Any, shape: tuple[int, ...], active: CompressionConfig, dtype: str) -> Any:
            return dequantize_tensor(payload, shape, active, dtype=dtype, extension_status=extension_status)

        return cls(config=config, quantize=quantize, dequantize=dequantize,
                   error_feedback=error_feedback or ErrorFeedbackState())

    @classmethod
    def from_hip_codec(cls, config: CompressionConfig, *, error_feedback: ErrorFeedbackState | None = None,
                       fused: bool = True) -> "DDPBucketProcessor":
        """Bind the GPU codec callables; ``fused`` runs the local round trip as one kernel per bucket."""
        from lowbit_comm_amd.hip.codec import FusedErrorFeedbackCodec, dequantize_tensor_hip, quantize_tensor_hip

        state = error_feedback or ErrorFeedbackState()
        return cls(config=config, quantize=quantize_tensor_hip, dequantize=dequantize_tensor_hip,
                   error_feedback=state,
                   fused_codec=FusedErrorFeedbackCodec(config, error_feedback=state) if fused else None)

    def process(self, bucket: Any, *, dtype: str) -> Any:
        key = bucket_key(bucket)
        original = bucket_tensor(bucket)
        use_feedback = self.config.error_feedback

        if self.all_reduce is None and self.fused_codec is not None:
            _payload, restored = self.fused_codec.step(key, original, dtype, update=use_feedback, apply=use_feedback)
            return restored

        prepared = self.error_feedback.compensate(key, original) if use_feedback else original
        shape = tuple(getattr(prepared, "shape", ()))
        if self.all_reduce is None:
            restored = self.dequantize(self.quantize(prepared, self.config), shape, self.config, dtype)
        else:
            restored = CompressedAllReduce(
                config=self.config,
                compress=lambda tensor, active: CompressedPayload(
                    buffer=self.quantize(tensor, active), shape=tuple(getattr(tensor, "shape", ())), dtype=dtype),
                all_reduce=self.all_reduce,
                decompress=lambda payload, active: self.dequantize(payload.buffer, payload.shape, active,
                                                                   payload.dtype),
            ).run(prepared, op="sum")
        if use_feedback:
            self.error_feedback.update(key, original=prepared, transmitted=restored)
        return restored
