"""Payload containers of the compression path, and the compressed all-reduce adapter.

``CompressedPayload`` has the reference's fields (``ccdl_comm/communication/collectives.py:11-22``);
``PackedPayload`` adds the one thing the GPU codec knows that the reference's type cannot say: that
codes and scales already sit in one allocation in wire order.
"""
from __future__ import annotations

import dataclasses
from collections.abc import Callable, Mapping
from typing import Any

from lowbit_comm_amd.config import CompressionConfig


@dataclasses.dataclass(frozen=True)
class CompressedPayload:
    """``buffer``: int8 codes (or packed bytes).  ``shape`` / ``dtype``: of the tensor it encodes
    (dtype as ``"fp16"`` / ``"bf16"`` / ``"fp32"``).  ``metadata`` for the linear INT8 codec:
    ``"scales"`` (float32, one per group) and ``"original_numel"``."""

    buffer: Any
    shape: tuple[int, ...]
    dtype: str
    metadata: Mapping[str, Any] = dataclasses.field(default_factory=dict)

    def with_buffer(self, buffer: Any) -> "CompressedPayload":
        """A copy around another buffer (e.g. the one a collective returned)."""
        return dataclasses.replace(self, buffer=buffer)

    @property
    def original_numel(self) -> int:
        """Element count of the encoded tensor (from the metadata, else from ``shape``)."""
        if "original_numel" in self.metadata:
            return int(self.metadata["original_numel"])
        count = 1
        for dim in self.shape:
            count *= int(dim)
        return count


@dataclasses.dataclass(frozen=True)
class PackedPayload(CompressedPayload):
    """``buffer`` and the tensor metadata are adjacent views of the ``uint8`` tensor ``packed``
    (``[codes || scales]``), so a byte collective can ship ``packed`` as is."""

    packed: Any = None

    @property
    def wire_bytes(self) -> int:
        """Bytes a collective has to move for this payload."""
        return int(self.packed.numel()) if self.packed is not None else 0


class CompressedAllReduce:
    """``decompress(all_reduce(compress(x), op))``.  The injected ``all_reduce`` owns the collective; this
    object only fixes the order of the three steps (``ccdl_comm/communication/collectives.py:25-41``)."""

    def __init__(self, config: CompressionConfig, compress: Callable[[Any, CompressionConfig], CompressedPayload],
                 all_reduce: Callable[[CompressedPayload, str], CompressedPayload],
                 decompress: Callable[[CompressedPayload, CompressionConfig], Any]) -> None:
        self.config = config
        self.compress = compress
        self.all_reduce = all_reduce
        self.decompress = decompress

    def run(self, tensor: Any, *, op: str = "sum") -> Any:
        sent = self.compress(tensor, self.config)
        returned = self.all_reduce(sent, op)
        return self.decompress(returned, self.config)
