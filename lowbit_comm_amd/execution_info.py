"""Diagnostics returned next to results (types of ``ccdl_comm/execution_info.py:14-110``)."""
from __future__ import annotations

import math
from collections.abc import Mapping
from dataclasses import dataclass, field
from types import MappingProxyType


def _non_empty(value: str, name: str) -> None:
    if not isinstance(value, str) or not value.strip():
        raise ValueError(f"{name} must be a non-empty string")


@dataclass(frozen=True)
class ExecutionInfo:
    """What ran: requested vs executed strategy, fallback and its reason, byte counts, fast path name."""

    requested_strategy: str
    executed_strategy: str
    backend: str
    fallback_used: bool
    fallback_reason: str | None
    stage_names: tuple[str, ...]
    original_bytes: int
    compressed_bytes: int
    compression_ratio: float
    workspace_cache_hit: bool
    async_capable: bool
    fast_path: str
    details: Mapping[str, object] = field(default_factory=dict)

    def __post_init__(self) -> None:
        for name in ("requested_strategy", "executed_strategy", "backend", "fast_path"):
            _non_empty(getattr(self, name), name)
        stages = tuple(self.stage_names)
        for stage in stages:
            _non_empty(stage, "stage name")
        object.__setattr__(self, "stage_names", stages)
        if self.original_bytes < 0:
            raise ValueError("original_bytes must be >= 0")
        if self.compressed_bytes < 0:
            raise ValueError("compressed_bytes must be >= 0")
        if not math.isfinite(self.compression_ratio) or self.compression_ratio <= 0.0:
            raise ValueError("compression_ratio must be finite and > 0")
        if self.fallback_used and not (self.fallback_reason or "").strip():
            raise ValueError("fallback_reason is required when fallback_used is true")
        if not self.fallback_used and self.fallback_reason is not None:
            raise ValueError("fallback_reason must be None when fallback_used is false")
        object.__setattr__(self, "details", MappingProxyType(dict(self.details)))


@dataclass(frozen=True)
class ExecutionCounterSnapshot:
    run_calls: int
    completed_runs: int
    failed_runs: int
    wait_calls: int
    query_calls: int


class ExecutionCounters:
    """Plain counters shared by an executor and its work objects (diagnostic, not synchronisation state)."""

    __slots__ = ("_run_calls", "_completed_runs", "_failed_runs", "_wait_calls", "_query_calls")

    def __init__(self) -> None:
        self._run_calls = self._completed_runs = self._failed_runs = self._wait_calls = self._query_calls = 0

    def snapshot(self) -> ExecutionCounterSnapshot:
        return ExecutionCounterSnapshot(self._run_calls, self._completed_runs, self._failed_runs,
                                        self._wait_calls, self._query_calls)

    def _record_run(self) -> None:
        self._run_calls += 1

    def _record_completed(self) -> None:
        self._completed_runs += 1

    def _record_failed(self) -> None:
        self._failed_runs += 1

    def _record_wait(self) -> None:
        self._wait_calls += 1

    def _record_query(self) -> None:
        self._query_calls += 1
