"""Gather-then-reduce adapter (``ccdl_comm/communication/gather_reduce.py:11-45``): every rank
receives all payloads, decodes them in rank order and adds them left to right."""
from __future__ import annotations

from collections.abc import Callable, Sequence
from dataclasses import dataclass
from typing import Any

from lowbit_comm_amd.config import CompressionConfig


@dataclass(frozen=True)
class GatheredPayloads:
    """What an all-gather of compressed payloads returns: one entry per rank, in rank order."""

    payloads: Sequence[Any]
    world_size: int


def sum_in_order(tensors: Sequence[Any]) -> Any:
    """``((t0 + t1) + t2) + ...`` - the order is part of the numerical contract."""
    if not tensors:
        raise ValueError("cannot reduce an empty payload list")
    total = tensors[0]
    for term in tensors[1:]:
        total = total + term
    return total


@dataclass(frozen=True)
class CompressedAllGatherReduce:
    config: CompressionConfig
    compress: Callable[[Any, CompressionConfig], Any]
    all_gather: Callable[[Any], GatheredPayloads]
    decompress: Callable[[Any, tuple[int, ...], CompressionConfig, str], Any]
    # Optional fused decode+reduce of all gathered payloads in one kernel.  Receives
    # (payloads, shape, config, dtype, reduce) and returns the reduced tensor, or None to decline.
    fused_decompress_reduce: Callable[..., Any] | None = None

    def run(self, tensor: Any, *, shape: tuple[int, ...], dtype: str, reduce: str = "mean") -> Any:
        if reduce not in ("mean", "sum"):
            raise ValueError(f"unsupported gather-reduce mode: {reduce}")
        gathered = self.all_gather(self.compress(tensor, self.config))
        if self.fused_decompress_reduce is not None:
            fused = self.fused_decompress_reduce(gathered.payloads, shape, self.config, dtype, reduce)
            if fused is not None:
                return fused
        total = sum_in_order([self.decompress(p, shape, self.config, dtype) for p in gathered.payloads])
        if reduce != "mean":
            return total
        if getattr(total, "is_cuda", False):     # torch divides GPU tensors by a Python number via the reciprocal
            from lowbit_comm_amd.hip.ops import true_divide_

            return true_divide_(total, gathered.world_size)
        return total / gathered.world_size
