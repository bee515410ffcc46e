"""Synchronous compressed bucket processing (``ccdl_comm/communication/ddp.py:33-97``).

``process`` runs ``compensate -> quantize -> [all_reduce] -> dequantize -> residual update`` for one
DDP bucket and never touches ``torch.distributed`` itself.  ``from_hip_codec`` binds the GPU codec;
with ``fused=True`` and no collective the whole local round trip is a single kernel.
"""
from __future__ import annotations

from collections.abc import Callable, Hashable
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


class DDPBucketProcessor:
    """One bucket at a time: ``compensate -> quantize -> [all_reduce] -> dequantize -> residual update``.

    ``quantize(tensor, config)`` and ``dequantize(payload, shape, config, dtype)`` are positional callables;
    ``all_reduce(payload, op)`` is optional (``None`` = local round trip); ``fused_codec`` (a
    ``FusedErrorFeedbackCodec``) replaces the whole local round trip by one kernel.
    """

    def __init__(self, config: CompressionConfig, quantize: Callable[[Any, CompressionConfig], Any],
                 dequantize: Callable[[Any, tuple[int, ...], CompressionConfig, str], Any],
                 all_reduce: Callable[[CompressedPayload, str], CompressedPayload] | None = None,
                 error_feedback: ErrorFeedbackState | None = None, fused_codec: Any | None = None) -> None:
        self.config = config
        self.quantize = quantize
        self.dequantize = dequantize
        self.all_reduce = all_reduce
        self.error_feedback = ErrorFeedbackState() if error_feedback is None else error_feedback
        self.fused_codec = fused_codec

    # ---- constructors ----------------------------------------------------------------------------
    @classmethod
    def from_cuda_codec(cls, config: CompressionConfig, *, extension_status: Any | None = None,
                        error_feedback: ErrorFeedbackState | None = None) -> "DDPBucketProcessor":
        """Codec facade with flat ``uint8`` buffers (the reference's constructor name)."""
        from lowbit_comm_amd.quantization import codec

        return cls(
            config,
            quantize=lambda tensor, active: codec.quantize_tensor(tensor, active, extension_status=extension_status),
            dequantize=lambda payload, shape, active, dtype: codec.dequantize_tensor(
                payload, shape, active, dtype=dtype, extension_status=extension_status),
            error_feedback=error_feedback,
        )

    @classmethod
    def from_hip_codec(cls, config: CompressionConfig, *, error_feedback: ErrorFeedbackState | None = None,
                       fused: bool = True) -> "DDPBucketProcessor":
        """GPU codec callables; with ``fused`` the local round trip is one kernel per bucket."""
        from lowbit_comm_amd.hip import codec as hip_codec

        state = ErrorFeedbackState() if error_feedback is None else error_feedback
        one_kernel = hip_codec.FusedErrorFeedbackCodec(config, error_feedback=state) if fused else None
        return cls(config, hip_codec.quantize_tensor_hip, hip_codec.dequantize_tensor_hip, error_feedback=state,
                   fused_codec=one_kernel)

    # ---- the step ----------------------------------------------------------------------------------
    def _round_trip(self, prepared: Any, dtype: str) -> Any:
        shape = tuple(getattr(prepared, "shape", ()))
        if self.all_reduce is None:
            return self.dequantize(self.quantize(prepared, self.config), shape, self.config, dtype)

        def compress(tensor: Any, active: CompressionConfig) -> CompressedPayload:
            return CompressedPayload(buffer=self.quantize(tensor, active), shape=tuple(getattr(tensor, "shape", ())),
                                     dtype=dtype)

        def decompress(payload: CompressedPayload, active: CompressionConfig) -> Any:
            return self.dequantize(payload.buffer, payload.shape, active, payload.dtype)

        return CompressedAllReduce(self.config, compress, self.all_reduce, decompress).run(prepared, op="sum")

    def process(self, bucket: Any, *, dtype: str) -> Any:
        key, original = bucket_key(bucket), bucket_tensor(bucket)
        feedback_on = self.config.error_feedback
        if self.all_reduce is None and self.fused_codec is not None:
            return self.fused_codec.step(key, original, dtype, update=feedback_on, apply=feedback_on)[1]
        prepared = self.error_feedback.compensate(key, original) if feedback_on else original
        restored = self._round_trip(prepared, dtype)
        if feedback_on:
            self.error_feedback.update(key, original=prepared, transmitted=restored)
        return restored
