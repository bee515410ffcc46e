"""What an executor reports next to its result: which path ran, why a fallback was taken, byte counts.

Same fields as the reference's ``ExecutionInfo`` / ``ExecutionCounters``
(``ccdl_comm/execution_info.py:14-110``); only the compression-path executors of this package fill them.
"""
from __future__ import annotations

import dataclasses
import math
from collections.abc import Mapping
from dataclasses import dataclass, field
from types import MappingProxyType

_NAMED = ("requested_strategy", "executed_strategy", "backend", "fast_path")
_EVENTS = ("run_calls", "completed_runs", "failed_runs", "wait_calls", "query_calls")


def _named(value: object, what: str) -> None:
    if not (isinstance(value, str) and value.strip()):
        raise ValueError(f"{what} must be a non-empty string")


@dataclass(frozen=True)
class ExecutionInfo:
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
        for name in _NAMED:
            _named(getattr(self, name), name)
        stages = tuple(self.stage_names)
        for stage in stages:
            _named(stage, "stage name")
        for name in ("original_bytes", "compressed_bytes"):
            if getattr(self, name) < 0:
                raise ValueError(f"{name} must be >= 0")
        ratio = self.compression_ratio
        if not (math.isfinite(ratio) and ratio > 0.0):
            raise ValueError("compression_ratio must be finite and > 0")
        has_reason = bool((self.fallback_reason or "").strip())
        if self.fallback_used and not has_reason:
            raise ValueError("fallback_reason is required when fallback_used is true")
        if not self.fallback_used and self.fallback_reason is not None:
            raise ValueError("fallback_reason must be None when fallback_used is false")
        object.__setattr__(self, "stage_names", stages)
        object.__setattr__(self, "details", MappingProxyType(dict(self.details)))

    # ---- conveniences used by this package's executors -------------------------------------------
    @classmethod
    def for_fused_path(cls, *, strategy: str, fast_path: str, stage: str, original_bytes: int,
                       compressed_bytes: int, backend: str = "hip") -> "ExecutionInfo":
        """Description of a single-stage fused execution with no fallback."""
        ratio = original_bytes / compressed_bytes if original_bytes > 0 and compressed_bytes > 0 else 1.0
        return cls(requested_strategy=strategy, executed_strategy=strategy, backend=backend, fallback_used=False,
                   fallback_reason=None, stage_names=(stage,), original_bytes=original_bytes,
                   compressed_bytes=compressed_bytes, compression_ratio=ratio, workspace_cache_hit=True,
                   async_capable=False, fast_path=fast_path)

    def with_fallback(self, reason: str, *, fast_path: str = "python_fallback") -> "ExecutionInfo":
        """The same execution, recorded as having taken a fallback for ``reason``."""
        return dataclasses.replace(self, fallback_used=True, fallback_reason=reason, fast_path=fast_path)

    def as_dict(self) -> dict[str, object]:
        """JSON-friendly form (``details`` copied into a plain dict)."""
        out = {f.name: getattr(self, f.name) for f in dataclasses.fields(self)}
        out["details"] = dict(self.details)
        out["stage_names"] = list(self.stage_names)
        return out


@dataclass(frozen=True)
class ExecutionCounterSnapshot:
    run_calls: int
    completed_runs: int
    failed_runs: int
    wait_calls: int
    query_calls: int


class ExecutionCounters:
    """Five plain integers shared by an executor and the work it hands out.  Diagnostic only: updates
    are unsynchronised increments, snapshots are best effort under concurrent use."""

    __slots__ = ("_counts",)

    def __init__(self) -> None:
        self._counts = [0] * len(_EVENTS)

    def snapshot(self) -> ExecutionCounterSnapshot:
        return ExecutionCounterSnapshot(*self._counts)

    def _bump(self, slot: int) -> None:
        self._counts[slot] += 1

    def _record_run(self) -> None:
        self._bump(0)

    def _record_completed(self) -> None:
        self._bump(1)

    def _record_failed(self) -> None:
        self._bump(2)

    def _record_wait(self) -> None:
        self._bump(3)

    def _record_query(self) -> None:
        self._bump(4)
