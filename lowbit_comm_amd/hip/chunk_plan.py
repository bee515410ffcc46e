"""Equal contiguous destination chunks of a flattened bucket
(plan of ``ccdl_comm/cuda/transports/compressed_reduce_scatter.py:72-94``)."""
from __future__ import annotations

from dataclasses import dataclass


def _integer(value: object, name: str) -> None:
    if isinstance(value, bool) or not isinstance(value, int):
        raise TypeError(f"{name} must be an integer")


@dataclass(frozen=True)
class ChunkRange:
    """Half-open range ``[start, stop)`` of the flattened tensor owned by one destination rank."""

    start: int
    stop: int

    def __post_init__(self) -> None:
        _integer(self.start, "chunk start")
        _integer(self.stop, "chunk stop")
        if self.start < 0:
            raise ValueError("chunk start must be >= 0")
        if self.stop < self.start:
            raise ValueError("chunk stop must be >= start")

    @property
    def numel(self) -> int:
        return self.stop - self.start


def _equal_ranges(shard_numel: int, world_size: int) -> tuple[ChunkRange, ...]:
    return tuple(ChunkRange(r * shard_numel, (r + 1) * shard_numel) for r in range(world_size))


@dataclass(frozen=True)
class ChunkPlan:
    original_numel: int
    world_size: int
    padded_numel: int
    shard_numel: int
    chunks: tuple[ChunkRange, ...]
    owner_by_chunk: tuple[int, ...]

    def __post_init__(self) -> None:
        for name in ("original_numel", "world_size", "padded_numel", "shard_numel"):
            _integer(getattr(self, name), name)
        if self.original_numel < 0:
            raise ValueError("original_numel must be >= 0")
        if self.world_size <= 0:
            raise ValueError("world_size must be > 0")
        if self.shard_numel < 0:
            raise ValueError("shard_numel must be >= 0")
        if self.padded_numel != self.shard_numel * self.world_size:
            raise ValueError("padded_numel must equal shard_numel * world_size")
        if self.padded_numel < self.original_numel:
            raise ValueError("padded_numel must be >= original_numel")
        if self.chunks != _equal_ranges(self.shard_numel, self.world_size):
            raise ValueError("chunks must be contiguous equal-sized rank ranges")
        for owner in self.owner_by_chunk:
            _integer(owner, "owner_by_chunk entry")
        if self.owner_by_chunk != tuple(range(self.world_size)):
            raise ValueError("owner_by_chunk must map each chunk to its destination rank")

    def chunk_for_rank(self, rank: int) -> ChunkRange:
        _integer(rank, "rank")
        if not 0 <= rank < self.world_size:
            raise ValueError(f"rank must be in [0, {self.world_size})")
        return self.chunks[rank]


def compile_chunk_plan(*, original_numel: int, world_size: int) -> ChunkPlan:
    """``shard_numel = ceil(n / W)``; the bucket is treated as zero padded to ``W * shard_numel``."""
    _integer(original_numel, "original_numel")
    _integer(world_size, "world_size")
    if original_numel < 0:
        raise ValueError("original_numel must be >= 0")
    if world_size <= 0:
        raise ValueError("world_size must be > 0")
    shard = -(-original_numel // world_size)
    return ChunkPlan(original_numel=original_numel, world_size=world_size, padded_numel=shard * world_size,
                     shard_numel=shard, chunks=_equal_ranges(shard, world_size),
                     owner_by_chunk=tuple(range(world_size)))
