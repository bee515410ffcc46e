"""What completes a DDP bucket whose all-gather ran asynchronously, as one object.

Counterpart of ``AsyncBucketPipeline`` (``ccdl_comm/communication/async_pipeline.py:10-65``): same keyword
arguments, same order of steps, same treatment of a failing step.  The comm hook builds one per bucket when
``async_gather`` and error feedback are both on."""
from __future__ import annotations

from collections.abc import Callable
from typing import Any


def chain_after(work: Any, finish: Callable[[Any], Any]) -> None:
    """Run ``finish`` once ``work`` is done: behind the work's own future when it offers one
    (``get_future().then``), immediately otherwise."""
    get_future = getattr(work, "get_future", None)
    inner = get_future() if callable(get_future) else None
    if inner is not None and hasattr(inner, "then"):
        inner.then(finish)
    else:
        finish(None)


class AsyncBucketPipeline:
    """``run()`` hangs the bucket's completion behind the gather and returns ``future``.  The completion waits for the
    gather, hands the gathered payloads to ``dequantize_reduce``, its result to ``update_feedback``, calls
    ``advance_policy``, orders the result on the device through ``completion_manager.record_for(result).wait()`` - and
    on the host too (``synchronize()``) unless ``synchronize_completion`` is false - and resolves ``future`` with the
    result.  A step that raises resolves the future with the exception when it has ``set_exception``; otherwise the
    exception propagates out of the completion."""

    def __init__(self, *, gather_work: Any, future: Any, dequantize_reduce: Callable[[Any], Any],
                 update_feedback: Callable[[Any], None], advance_policy: Callable[[], None],
                 completion_manager: Any | None = None, synchronize_completion: bool = True) -> None:
        if completion_manager is None:
            from lowbit_comm_amd.hip.workspace import EventCompletionManager

            completion_manager = EventCompletionManager()
        self._work = gather_work
        self._future = future
        self._decode = dequantize_reduce
        self._update = update_feedback
        self._advance = advance_policy
        self._completions = completion_manager
        self._host_wait = bool(synchronize_completion)

    def run(self) -> Any:
        chain_after(self._work, self._complete)
        return self._future

    def _complete(self, _unused: Any = None) -> Any:
        try:
            restored = self._decode(self._work.wait())
            self._update(restored)
            self._advance()
            done = self._completions.record_for(restored)
            done.wait()
            block_host = getattr(done, "synchronize", None)
            if self._host_wait and callable(block_host):
                block_host()
        except Exception as exc:
            carry = getattr(self._future, "set_exception", None)
            if not callable(carry):
                raise
            carry(exc)
            return None
        self._future.set_result(restored)
        return restored


__all__ = ["AsyncBucketPipeline", "chain_after"]
