"""Asynchronous results of compressed collectives: a handle to wait on, a deferred host-side completion step and a
device-side completion, behind one ``wait() / query()`` object.

Mirrors the work objects of the reference: the Python ``CompletionWork`` (``ccdl_comm/work.py:58-190``) and the
native ``CompressedWork`` (``ccdl_comm/csrc/executor/compressed_work.cpp:8-228``), whose stronger guarantees are the
ones kept here: ``wait()`` may be called from several threads, the transport wait and the completion callback run
exactly once, every waiter sees the same result or the same exception object, and the device-side completion is
a stream wait, not a host synchronisation, whenever the completion offers one.
"""
from __future__ import annotations

import threading
from dataclasses import replace
from typing import Any, Callable, Sequence

from lowbit_comm_amd.execution_info import ExecutionCounters, ExecutionInfo


def _call(target: Any, name: str) -> bool:
    method = getattr(target, name, None)
    if callable(method):
        method()
        return True
    return False


def is_done(target: Any) -> bool:
    """Non-blocking completion test of a foreign handle: ``None`` is done, ``is_completed()`` or ``query()``
    decide otherwise, an object with neither is treated as pending (compressed_work.cpp:43-54)."""
    if target is None:
        return True
    for name in ("is_completed", "query"):
        probe = getattr(target, name, None)
        if callable(probe):
            return bool(probe())
    return False


class CollectiveWork:
    """Protocol of an asynchronous collective result."""

    execution_info: ExecutionInfo | None = None
    execution_counters: ExecutionCounters | None = None

    def wait(self) -> Any:
        raise NotImplementedError

    def query(self) -> bool:
        raise NotImplementedError

    def get_future(self) -> Any | None:
        return None

    def result(self) -> Any:
        return self.wait()


class ImmediateWork(CollectiveWork):
    """A result that is already there, behind the same interface."""

    def __init__(self, value: Any, *, execution_info: ExecutionInfo | None = None,
                 execution_counters: ExecutionCounters | None = None) -> None:
        self._value = value
        self.execution_info = execution_info
        self.execution_counters = execution_counters
        if execution_counters is not None:
            execution_counters._record_completed()

    def wait(self) -> Any:
        if self.execution_counters is not None:
            self.execution_counters._record_wait()
        return self._value

    def query(self) -> bool:
        if self.execution_counters is not None:
            self.execution_counters._record_query()
        return True


_PENDING, _RUNNING, _DONE = 0, 1, 2


class CompletionWork(CollectiveWork):
    """``handle`` (a transport's work: ``wait`` / ``is_completed``), then ``complete()`` (host-side step that
    produces the result, e.g. the fused decode of what the transport delivered), then ``completion`` (device-side:
    ``wait()`` orders the caller's current stream after it).  ``resources`` are kept referenced while in flight."""

    def __init__(self, result: Any, *, handle: Any | None = None, complete: Callable[[], Any] | None = None,
                 completion: Any | None = None, resources: Sequence[Any] = (),
                 execution_info: ExecutionInfo | None = None,
                 execution_counters: ExecutionCounters | None = None) -> None:
        self._value = result
        self._handle = handle
        self._complete = complete
        self._completion = completion
        self._resources = tuple(resources)
        self._state = _PENDING
        self._callback_pending = complete is not None
        self._error: BaseException | None = None
        self._lock = threading.Lock()
        self._finished = threading.Event()
        self.execution_info = execution_info
        self.execution_counters = execution_counters

    @property
    def resources(self) -> tuple[Any, ...]:
        return self._resources

    def query(self) -> bool:
        """Non-blocking: transport first, then the callback (which only ``wait`` runs), then the completion."""
        if self.execution_counters is not None:
            self.execution_counters._record_query()
        if self._state == _DONE:
            return True
        if not is_done(self._handle) or self._callback_pending:
            return False
        return is_done(self._completion)

    def wait(self) -> Any:
        if self.execution_counters is not None:
            self.execution_counters._record_wait()
        with self._lock:
            first = self._state == _PENDING
            if first:
                self._state = _RUNNING
        if first:
            try:
                _call(self._handle, "wait")
                if self._callback_pending:
                    self._callback_pending = False          # a failing callback is not retried
                    self._value = self._complete()
                if not _call(self._completion, "wait"):      # a stream wait where there is one ...
                    _call(self._completion, "synchronize")   # ... a host wait only as the last resort
            except BaseException as error:                   # cached: every waiter gets this object
                self._error = error
            self._complete = None
            self._state = _DONE
            if self.execution_counters is not None:
                (self.execution_counters._record_failed if self._error is not None
                 else self.execution_counters._record_completed)()
            self._finished.set()
        else:
            self._finished.wait()
        if self._error is not None:
            raise self._error
        return self._value

    def get_future(self) -> Any | None:
        future = getattr(self._handle, "get_future", None)
        return future() if callable(future) else None

    def release_resources(self) -> None:
        """Drop the references to in-flight buffers; only valid once the work is done."""
        if self._state != _DONE:
            raise RuntimeError("resources of unfinished work cannot be released")
        self._resources = ()


def python_fallback_info(info: ExecutionInfo | None) -> ExecutionInfo | None:
    """Metadata of work that runs through this module rather than a native executor."""
    return None if info is None else replace(info, fast_path="python_fallback")
