"""A rank-local reduced shard with the bookkeeping needed to place it back into the original tensor.

Field names and derived quantities match the reference's ``ReducedShard`` (``ccdl_comm/shard.py:12-97``)
so results can be handed to code written against it.
"""
from __future__ import annotations

from collections.abc import Mapping
from dataclasses import dataclass, field, fields
from types import MappingProxyType
from typing import Any

_EXPORTED = ("shard_index", "shard_numel", "shard_offset", "shard_end", "valid_numel", "original_shape",
             "original_numel", "padded_numel", "world_size", "reduce", "dtype", "layout", "transport")


def _check_geometry(index: int, per_shard: int, total: int, world: int, padded: int | None) -> int:
    """Validate the shard geometry and return the padded element count (``world * per_shard``)."""
    problems = (
        (world <= 0, "world_size must be > 0"),
        (index < 0, "shard_index must be >= 0"),
        (world > 0 and index >= world, "shard_index must be < world_size"),
        (per_shard < 0, "shard_numel must be >= 0"),
        (total < 0, "original_numel must be >= 0"),
    )
    for failed, message in problems:
        if failed:
            raise ValueError(message)
    whole = per_shard * world
    claimed = whole if padded is None else padded
    if claimed < total:
        raise ValueError("padded_numel must be >= original_numel")
    if claimed != whole:
        raise ValueError("padded_numel must equal shard_numel * world_size")
    return claimed


@dataclass(frozen=True)
class ReducedShard:
    """``shard`` holds elements ``[shard_index * shard_numel, ...)`` of the zero-padded flattened tensor."""

    shard: Any
    shard_index: int
    shard_numel: int
    original_shape: tuple[int, ...]
    original_numel: int
    world_size: int
    reduce: str
    padded_numel: int | None = None
    dtype: str = "auto"
    layout: str = "flat_contiguous"
    transport: str = "unknown"
    metadata: Mapping[str, Any] = field(default_factory=dict)

    def __post_init__(self) -> None:
        padded = _check_geometry(self.shard_index, self.shard_numel, self.original_numel, self.world_size,
                                 self.padded_numel)
        dims = tuple(self.original_shape)
        for dim in dims:
            if type(dim) is not int or dim < 0:
                raise ValueError("original_shape dimensions must be non-negative integers")
        frozen = {"original_shape": dims, "padded_numel": padded, "metadata": MappingProxyType(dict(self.metadata))}
        for name, value in frozen.items():
            object.__setattr__(self, name, value)

    # ---- where the shard sits in the unpadded tensor --------------------------------------------
    @property
    def shard_offset(self) -> int:
        return self.shard_numel * self.shard_index

    @property
    def shard_end(self) -> int:
        return min(self.original_numel, self.shard_offset + self.shard_numel)

    @property
    def logical_range(self) -> tuple[int, int]:
        return (self.shard_offset, self.shard_end)

    @property
    def valid_numel(self) -> int:
        start, stop = self.logical_range
        return stop - start if stop > start else 0

    @property
    def padding_numel(self) -> int:
        return self.shard_numel - self.valid_numel

    @property
    def is_padding_only(self) -> bool:
        return self.valid_numel == 0

    @property
    def has_padding(self) -> bool:
        return self.padding_numel > 0 or int(self.padded_numel or 0) > self.original_numel

    def to_metadata(self) -> dict[str, Any]:
        """Plain-dict description (everything except the tensor itself)."""
        described = {name: getattr(self, name) for name in _EXPORTED}
        described["metadata"] = dict(self.metadata)
        return described


assert {f.name for f in fields(ReducedShard)} >= {"shard", "metadata", "reduce"}
