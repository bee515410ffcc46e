"""MI355X-native compression data path for DDP gradient communication.

The package mirrors the reference library's surface for this path - ``CompressionConfig``, the
``quantize_tensor`` / ``dequantize_tensor`` facade and ``Quantizer``, ``CompressedPayload`` and the
fused-payload packer, ``DDPBucketProcessor`` and ``create_ddp_comm_hook``, the workspace pool - over
hand-written gfx950 kernels behind a C ABI (``include/lbc.h``).  Importing it needs neither a GPU nor
the built library; using the codec does.
"""
from .config import CompressionConfig
from .exceptions import CCDLError, CCDLUnavailableError, UnsupportedCollective
from .execution_info import ExecutionCounters, ExecutionCounterSnapshot, ExecutionInfo
from .shard import ReducedShard
from .work import CollectiveWork, CompletionWork, ImmediateWork

__all__ = [
    "CCDLError", "CCDLUnavailableError", "CollectiveWork", "CompletionWork", "CompressionConfig",
    "ExecutionCounterSnapshot", "ExecutionCounters", "ExecutionInfo", "ImmediateWork", "Quantizer", "ReducedShard", "UnsupportedCollective", "dequantize_tensor",
    "estimate_quantized_size", "quantize_tensor",
]


def __getattr__(name: str):
    # the quantization facade imports lazily so that `import lowbit_comm_amd` stays torch-free
    if name in ("Quantizer", "dequantize_tensor", "estimate_quantized_size", "quantize_tensor",
                "estimate_payload_size"):
        from . import quantization

        return getattr(quantization, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
