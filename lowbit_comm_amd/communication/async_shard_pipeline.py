"""What happens after an asynchronous shard exchange has been started: wait for the payloads, reduce them to this
rank's shard, update error feedback, advance the policy, order the result on the device, hand back the workspaces
and complete the bucket's future - in that order, once, whether the exchange offers a future to chain on or not.

Counterpart of ``AsyncShardPipeline`` (``ccdl_comm/communication/async_shard_pipeline.py:11-129``), which the
reference's reduce-scatter transport returns for ``async_op=True``
(``ccdl_comm/communication/reduce_scatter_transport.py:286-333``); the order of the steps is the one its tests pin
(``tests/test_async_shard_pipeline.py:73-241``).
"""
from __future__ import annotations

from dataclasses import replace
from typing import Any, Callable, Sequence

from lowbit_comm_amd.shard import ReducedShard


def _default_completion_manager() -> Any:
    from lowbit_comm_amd.hip.completion import HipCompletionManager

    return HipCompletionManager()


class AsyncShardPipeline:
    """``run()`` chains the completion step on the exchange's future when it has one (``get_future().then``), else
    runs it at once; the pipeline itself is the work object the caller keeps: ``wait()``, ``query()``,
    ``get_future()``, ``then()``, ``resources``.

    ``reduce_shard(received) -> ReducedShard``, ``update_feedback(shard)`` and ``advance_policy()`` are the
    transport's callbacks.  ``workspace_leases`` are released with the completion recorded for the reduced shard
    (after that completion has been ordered), also when a callback fails - then with a completion recorded for the
    first lease's buffer - and the failure is delivered through the future.  ``resources`` are only kept alive."""

    def __init__(self, *, communication_work: Any, future: Any, reduce_shard: Callable[[Any], ReducedShard],
                 update_feedback: Callable[[ReducedShard], None], advance_policy: Callable[[], None],
                 completion_manager: Any | None = None, synchronize_completion: bool = False,
                 resources: Sequence[Any] = (), workspace_leases: Sequence[Any] = ()) -> None:
        self._exchange = communication_work
        self._outer = future
        self._reduce = reduce_shard
        self._feedback = update_feedback
        self._advance = advance_policy
        self._completions = completion_manager if completion_manager is not None else _default_completion_manager()
        self._host_wait = bool(synchronize_completion)
        self._kept = tuple(resources)
        self._leases = list(workspace_leases)

    # ---- start --------------------------------------------------------------------------------- #
    def run(self) -> "AsyncShardPipeline":
        source = getattr(self._exchange, "get_future", None)
        inner = source() if callable(source) else None
        if inner is not None and hasattr(inner, "then"):
            inner.then(self._finish)
        else:
            self._finish()
        return self

    # ---- the work-object face ------------------------------------------------------------------ #
    @property
    def resources(self) -> tuple[Any, ...]:
        return self._kept

    def get_future(self) -> Any:
        return self._outer

    def then(self, callback: Callable[[Any], Any]) -> Any:
        chain = getattr(self._outer, "then", None)
        if not callable(chain):
            raise AttributeError("underlying future does not support then()")
        return chain(callback)

    def query(self) -> bool:
        done = getattr(self._outer, "done", None)
        if callable(done):
            return bool(done())
        return any(getattr(self._outer, name, None) is not None for name in ("result", "exception"))

    def wait(self) -> ReducedShard:
        wait = getattr(self._outer, "wait", None)
        if callable(wait):
            return wait()
        failure = getattr(self._outer, "exception", None)
        if failure is not None:
            raise failure
        value = getattr(self._outer, "result", None)
        if value is None:
            raise RuntimeError("asynchronous shard result is not complete")
        return value

    # ---- completion step ----------------------------------------------------------------------- #
    def _give_back(self, completion: Any) -> None:
        while self._leases:
            self._leases.pop(0).release(completion=completion)

    def _finish(self, _inner_future: Any = None) -> ReducedShard | None:
        try:
            received = self._exchange.wait()
            reduced = self._reduce(received)
            shard = replace(reduced, metadata={**reduced.metadata, "async_completion": True})
            self._feedback(shard)
            self._advance()
            ordered = self._completions.record_for(shard.shard)
            ordered.wait()
            self._give_back(ordered)
            if self._host_wait:
                block = getattr(ordered, "synchronize", None)
                if callable(block):
                    block()
            self._outer.set_result(shard)
            return shard
        except Exception as failure:
            if self._leases:
                ordered = self._completions.record_for(getattr(self._leases[0], "buffer", None))
                ordered.wait()
                self._give_back(ordered)
            deliver = getattr(self._outer, "set_exception", None)
            if not callable(deliver):
                raise
            deliver(failure)
            return None
