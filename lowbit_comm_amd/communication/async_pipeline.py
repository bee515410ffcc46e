"""Completion of one bucket whose gather was started asynchronously.

Role of ``ccdl_comm/communication/async_pipeline.py:11-65``: once the gather work is done, decode and
reduce, update the error-feedback residual, advance the feedback policy, order the result on the device
and resolve the bucket's future.  Every step is a callable handed in by the hook, so this class only fixes
the order and where an exception goes (to the future, when it can carry one).
"""
from __future__ import annotations

from collections.abc import Callable
from typing import Any


class AsyncBucketPipeline:
    def __init__(self, *, gather_work: Any, future: Any, dequantize_reduce: Callable[[Any], Any],
                 update_feedback: Callable[[Any], None], advance_policy: Callable[[], None],
                 completion_manager: Any | None = None, synchronize_completion: bool = True) -> None:
        if completion_manager is None:
            from lowbit_comm_amd.hip.workspace import EventCompletionManager

            completion_manager = EventCompletionManager()
        self._work = gather_work
        self._future = future
        self._steps = (dequantize_reduce, update_feedback, advance_policy)
        self._manager = completion_manager
        self._synchronize = synchronize_completion

    def run(self) -> Any:
        """Chain the completion behind the gather's own future when it has one; else complete now."""
        get_future = getattr(self._work, "get_future", None)
        inner = get_future() if callable(get_future) else None
        if inner is not None and hasattr(inner, "then"):
            inner.then(self._complete)
        else:
            self._complete()
        return self._future

    def _complete(self, _unused: Any = None) -> Any:
        decode, update, advance = self._steps
        try:
            restored = decode(self._work.wait())
            update(restored)
            advance()
            done = self._manager.record_for(restored)
            done.wait()
            host_wait = getattr(done, "synchronize", None)
            if self._synchronize and callable(host_wait):
                host_wait()
        except Exception as exc:
            fail = getattr(self._future, "set_exception", None)
            if not callable(fail):
                raise
            fail(exc)
            return None
        self._future.set_result(restored)
        return restored
