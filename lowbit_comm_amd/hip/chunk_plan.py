"""Equal contiguous destination chunks of a flattened bucket
(plan of ``ccdl_comm/cuda/transports/compressed_reduce_scatter.py:72-94``)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import NamedTuple


def _integer(value: object, name: str) -> None:
    if isinstance(value, bool) or not isinstance(value, int):
        raise TypeError(f"{name} must be an integer")


class _Floor(NamedTuple):
    """``field`` must not be below ``lowest``; ``text`` is what the error says."""

    field: str
    lowest: int
    text: str


@dataclass(frozen=True)
class ChunkRange:
    """Half-open range ``[start, stop)`` of the flattened tensor owned by one destination rank."""

    start: int
    stop: int

    def __post_init__(self) -> None:
        for label in ("start", "stop"):
            _integer(getattr(self, label), f"chunk {label}")
        if self.start < 0:
            raise ValueError("chunk start must be >= 0")
        if self.start > self.stop:
            raise ValueError("chunk stop must be >= start")

    @property
    def numel(self) -> int:
        return self.stop - self.start


def _equal_ranges(shard_numel: int, world_size: int) -> tuple[ChunkRange, ...]:
    edges = range(0, (world_size + 1) * shard_numel, shard_numel) if shard_numel else [0] * (world_size + 1)
    return tuple(ChunkRange(a, b) for a, b in zip(edges, list(edges)[1:]))


_PLAN_FLOORS = (_Floor("original_numel", 0, "must be >= 0"), _Floor("world_size", 1, "must be > 0"),
                _Floor("shard_numel", 0, "must be >= 0"))


@dataclass(frozen=True)
class ChunkPlan:
    """Rank ``r`` owns ``chunks[r]``; the bucket counts as zero padded to ``padded_numel``.  Only the plan
    :func:`compile_chunk_plan` would build for the same sizes is accepted."""

    original_numel: int
    world_size: int
    padded_numel: int
    shard_numel: int
    chunks: tuple[ChunkRange, ...]
    owner_by_chunk: tuple[int, ...]

    def __post_init__(self) -> None:
        for name in ("original_numel", "world_size", "padded_numel", "shard_numel"):
            _integer(getattr(self, name), name)
        for floor in _PLAN_FLOORS:
            if getattr(self, floor.field) < floor.lowest:
                raise ValueError(f"{floor.field} {floor.text}")
        if self.shard_numel * self.world_size != self.padded_numel:
            raise ValueError("padded_numel must equal shard_numel * world_size")
        if self.original_numel > self.padded_numel:
            raise ValueError("padded_numel must be >= original_numel")
        if self.chunks != _equal_ranges(self.shard_numel, self.world_size):
            raise ValueError("chunks must be contiguous equal-sized rank ranges")
        for owner in self.owner_by_chunk:
            _integer(owner, "owner_by_chunk entry")
        if self.owner_by_chunk != tuple(range(self.world_size)):
            raise ValueError("owner_by_chunk must map each chunk to its destination rank")

    def chunk_for_rank(self, rank: int) -> ChunkRange:
        _integer(rank, "rank")
        if rank not in range(self.world_size):
            raise ValueError(f"rank must be in [0, {self.world_size})")
        return self.chunks[rank]


def compile_chunk_plan(*, original_numel: int, world_size: int) -> ChunkPlan:
    """``shard_numel = ceil(n / W)``; the bucket is treated as zero padded to ``W * shard_numel``."""
    for name, value in (("original_numel", original_numel), ("world_size", world_size)):
        _integer(value, name)
    for floor in _PLAN_FLOORS[:2]:
        if {"original_numel": original_numel, "world_size": world_size}[floor.field] < floor.lowest:
            raise ValueError(f"{floor.field} {floor.text}")
    shard = -(-original_numel // world_size)
    return ChunkPlan(original_numel=original_numel, world_size=world_size, padded_numel=shard * world_size,
                     shard_numel=shard, chunks=_equal_ranges(shard, world_size),
                     owner_by_chunk=tuple(range(world_size)))
