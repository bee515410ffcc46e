"""Adapters between DDP buckets, the codec and injected collectives."""
from .async_pipeline import AsyncBucketPipeline
from .async_shard_pipeline import AsyncShardPipeline
from .collectives import CompressedAllReduce, CompressedPayload, PackedPayload
from .gather_reduce import CompressedAllGatherReduce, GatheredPayloads
from .payload_packing import (
    DEFAULT_FUSED_PAYLOAD_MIN_NUMEL,
    FusedPayloadAllGather,
    FusedPayloadPacker,
    TensorFieldSchema,
    make_fused_payload_all_gather,
    make_payload_all_gather,
    should_fuse_payload,
)

__all__ = [
    "AsyncBucketPipeline", "AsyncShardPipeline", "CompressedAllGatherReduce", "CompressedAllReduce", "CompressedPayload", "DEFAULT_FUSED_PAYLOAD_MIN_NUMEL",
    "FusedPayloadAllGather", "FusedPayloadPacker", "GatheredPayloads", "PackedPayload", "TensorFieldSchema",
    "make_fused_payload_all_gather", "make_payload_all_gather", "should_fuse_payload",
]
