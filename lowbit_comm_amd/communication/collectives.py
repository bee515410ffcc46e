"""Payload container and the compress -> transport -> decompress adapter
(types of ``ccdl_comm/communication/collectives.py:11-41``)."""
from __future__ import annotations

from collections.abc import Callable, Mapping
from dataclasses import dataclass, field, replace
from typing import Any

from lowbit_comm_amd.config import CompressionConfig


@dataclass(frozen=True)
class CompressedPayload:
    """A compressed tensor: ``buffer`` (int8 codes or packed bytes) plus what is needed to rebuild it.

    For the linear INT8 codec ``metadata`` holds ``"scales"`` (float32, one per group) and
    ``"original_numel"`` (int).
    """

    buffer: Any
    shape: tuple[int, ...]
    dtype: str
    metadata: Mapping[str, Any] = field(default_factory=dict)

    def with_buffer(self, buffer: Any) -> "CompressedPayload":
        """Same shape, dtype and metadata around another buffer."""
        return replace(self, buffer=buffer)


@dataclass(frozen=True)
class PackedPayload(CompressedPayload):
    """A payload whose ``buffer`` and tensor metadata are adjacent views of one ``uint8`` allocation,
    ``packed``, already in wire order - packing it for a byte collective needs no copy."""

    packed: Any = None


@dataclass(frozen=True)
class CompressedAllReduce:
    """Order of operations of a compressed all-reduce; the injected ``all_reduce`` owns the collective."""

    config: CompressionConfig
    compress: Callable[[Any, CompressionConfig], CompressedPayload]
    all_reduce: Callable[[CompressedPayload, str], CompressedPayload]
    decompress: Callable[[CompressedPayload, CompressionConfig], Any]

    def run(self, tensor: Any, *, op: str = "sum") -> Any:
        return self.decompress(self.all_reduce(self.compress(tensor, self.config), op), self.config)
