"""Work objects and the completion manager (lowbit_comm_amd/work.py, lowbit_comm_amd/hip/completion.py) without a
GPU: ordering of transport wait, completion callback and device completion; wait-once under concurrency; cached
errors; stream work with a stand-in for torch.cuda.  Behaviour follows the reference's own tests for these objects
(tests/test_cuda_completion.py:39-260, tests/cuda/test_native_work.py:86-257)."""
import threading
import time

import pytest

from lowbit_comm_amd.execution_info import ExecutionCounters, ExecutionInfo
from lowbit_comm_amd.hip.completion import HipCompletionManager, HipStreamWork
from lowbit_comm_amd.hip.workspace import NoopCompletion
from lowbit_comm_amd.work import CompletionWork, ImmediateWork, is_done

INFO = ExecutionInfo(requested_strategy="reduce_scatter", executed_strategy="reduce_scatter", backend="hip",
                     fallback_used=False, fallback_reason=None, stage_names=(), original_bytes=8, compressed_bytes=2,
                     compression_ratio=4.0, workspace_cache_hit=True, async_capable=True, fast_path="hip_reduce_scatter")


class Handle:
    def __init__(self, log, done=False):
        self.log, self.done = log, done

    def wait(self):
        self.log.append("handle.wait")
        self.done = True

    def is_completed(self):
        self.log.append("handle.is_completed")
        return self.done


class Completion:
    def __init__(self, log, ready=True):
        self.log, self.ready = log, ready

    def wait(self):
        self.log.append("completion.wait")

    def synchronize(self):
        self.log.append("completion.synchronize")

    def query(self):
        self.log.append("completion.query")
        return self.ready


def test_wait_runs_transport_then_callback_then_completion_exactly_once():
    log = []
    work = CompletionWork("pending", handle=Handle(log), complete=lambda: log.append("complete") or "finished",
                          completion=Completion(log))
    assert work.query() is False and log == ["handle.is_completed"]      # non-blocking, transport asked first
    assert work.wait() == "finished" and work.wait() == "finished" and work.result() == "finished"
    assert log == ["handle.is_completed", "handle.wait", "complete", "completion.wait"]   # stream wait, no host sync
    assert work.query() is True and log[-1] == "completion.wait"         # a finished work asks nobody


def test_query_reports_pending_until_the_callback_has_run():
    log = []
    work = CompletionWork(None, handle=Handle(log, done=True), complete=lambda: 5, completion=Completion(log))
    assert work.query() is False                 # transport done, but only wait() runs the callback
    assert "completion.query" not in log
    assert work.wait() == 5 and work.query() is True
    plain = CompletionWork(7, completion=Completion(log, ready=False))
    assert plain.query() is False and plain.wait() == 7 and plain.query() is True


def test_completion_without_a_stream_wait_falls_back_to_synchronize():
    log = []

    class HostOnly:
        def synchronize(self):
            log.append("synchronize")

    assert CompletionWork(1, completion=HostOnly()).wait() == 1 and log == ["synchronize"]
    assert is_done(None) and not is_done(object())


def test_errors_are_cached_and_the_callback_is_not_retried():
    calls = []
    error = RuntimeError("post-processing failed")

    def fail():
        calls.append("complete")
        raise error

    counters = ExecutionCounters()
    work = CompletionWork(None, complete=fail, execution_counters=counters)
    for _ in range(3):
        with pytest.raises(RuntimeError) as caught:
            work.wait()
        assert caught.value is error
    assert calls == ["complete"] and work.query() is True
    snapshot = counters.snapshot()
    assert snapshot.failed_runs == 1 and snapshot.completed_runs == 0 and snapshot.wait_calls == 3

    class BrokenTransport:
        def wait(self):
            raise ValueError("link down")

    work = CompletionWork("x", handle=BrokenTransport(), complete=lambda: calls.append("never"))
    with pytest.raises(ValueError, match="link down"):
        work.wait()
    with pytest.raises(ValueError, match="link down"):
        work.wait()
    assert "never" not in calls


def test_concurrent_waiters_share_one_execution():
    calls = []
    gate = threading.Event()

    def slow():
        calls.append("complete")
        gate.wait(5)
        return "done"

    work = CompletionWork(None, complete=slow)
    results, errors = [], []

    def waiter():
        try:
            results.append(work.wait())
        except BaseException as error:      # pragma: no cover - reported below
            errors.append(error)

    threads = [threading.Thread(target=waiter) for _ in range(8)]
    for thread in threads:
        thread.start()
    time.sleep(0.05)
    assert calls == ["complete"] and not results            # one runs it, seven wait for it
    gate.set()
    for thread in threads:
        thread.join(5)
    assert not errors and results == ["done"] * 8 and calls == ["complete"]

    failing_calls = []

    def failing():
        failing_calls.append(1)
        time.sleep(0.02)
        raise KeyError("boom")

    work = CompletionWork(None, complete=failing)
    caught = []
    threads = [threading.Thread(target=lambda: caught.append(pytest.raises(KeyError, work.wait).value)) for _ in range(6)]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join(5)
    assert len(failing_calls) == 1 and len(caught) == 6 and len({id(e) for e in caught}) == 1


def test_resources_stay_referenced_until_released_after_completion():
    resource = object()
    work = CompletionWork(3, resources=(resource,), complete=lambda: 4)
    assert resource in work.resources
    with pytest.raises(RuntimeError, match="unfinished"):
        work.release_resources()
    assert work.wait() == 4 and resource in work.resources
    work.release_resources()
    assert work.resources == ()


def test_manager_builds_the_cheapest_work_that_fits():
    manager = HipCompletionManager(torch_provider=lambda: None)
    counters = ExecutionCounters()
    immediate = manager.create_work(result=9, execution_info=INFO, execution_counters=counters)
    assert isinstance(immediate, ImmediateWork) and immediate.query() and immediate.wait() == 9
    assert immediate.execution_info.fast_path == "hip_reduce_scatter" and counters.snapshot().completed_runs == 1
    callbacks = []
    ready = type("Ready", (), {"is_completed": lambda self: True, "wait": lambda self: None})()
    work = manager.create_work(result=None, handle=ready, complete=lambda: callbacks.append("complete") or 5,
                               execution_info=INFO, execution_counters=ExecutionCounters())
    assert isinstance(work, CompletionWork) and work.query() is False and callbacks == []
    assert work.execution_info.fast_path == "python_fallback"
    assert work.execution_info.requested_strategy == INFO.requested_strategy
    assert work.wait() == 5 and callbacks == ["complete"]
    assert work.get_future() is None
    with_future = manager.create_work(result=1, handle=type("H", (), {"get_future": lambda self: "future"})())
    assert with_future.get_future() == "future"


def test_manager_without_a_gpu_hands_out_noop_completions():
    manager = HipCompletionManager(torch_provider=lambda: None)
    assert isinstance(manager.create_stream_work(async_op=True), NoopCompletion)
    host_tensor = type("T", (), {"is_cuda": False})()
    completion = manager.record_for(host_tensor)
    assert isinstance(completion, NoopCompletion) and completion.query()
    completion.wait()
    completion.wait_stream("any")
    completion.synchronize()


class FakeCuda:
    """Stand-in for torch.cuda that logs every ordering call."""

    def __init__(self):
        self.log = []
        outer = self

        class Stream:
            def __init__(self, index):
                self.index = index

            def wait_stream(self, other):
                outer.log.append(("wait_stream", self.index, other.index))

            def wait_event(self, event):
                outer.log.append(("wait_event", self.index))

        class Guard:
            def __init__(self, stream):
                self.stream = stream

            def __enter__(self):
                outer.log.append(("enter", self.stream.index))

            def __exit__(self, *exc):
                outer.log.append(("exit", self.stream.index))

        class Event:
            def record(self, stream=None):
                outer.log.append(("record", None if stream is None else stream.index))

            def wait(self):
                outer.log.append("event.wait")

            def query(self):
                outer.log.append("event.query")
                return True

            def synchronize(self):
                outer.log.append("event.synchronize")

        self.StreamType, self.Event, self._guard = Stream, Event, Guard

    def is_available(self):
        return True

    def current_device(self):
        return 3

    def current_stream(self):
        return self.StreamType("current")

    def Stream(self, device):
        self.log.append(("new_stream", device))
        return self.StreamType(f"side{device}")

    def stream(self, stream):
        return self._guard(stream)


def test_stream_work_orders_the_side_stream_after_the_current_one_and_records_an_event(monkeypatch):
    from lowbit_comm_amd.hip import completion as completion_module

    monkeypatch.setattr(completion_module, "_COMMUNICATION_STREAMS", {})
    cuda = FakeCuda()
    torch_like = type("Torch", (), {"cuda": cuda})
    manager = HipCompletionManager(torch_provider=lambda: torch_like)
    handle_log = []
    work = manager.create_stream_work(async_op=True, handle=Handle(handle_log))
    assert isinstance(work, HipStreamWork)
    with work:
        cuda.log.append("body")
    assert work.query() is True
    work.wait()
    work.wait_stream(cuda.StreamType("other"))
    assert cuda.log == [("new_stream", 3), ("wait_stream", "side3", "current"), ("enter", "side3"), "body",
                        ("exit", "side3"), ("record", "side3"), "event.query", "event.wait", ("wait_event", "other")]
    assert handle_log == ["handle.wait"]
    # a second asynchronous work reuses the device's side stream; a synchronous one stays on the current stream
    cuda.log.clear()
    with manager.create_stream_work(async_op=True):
        pass
    assert ("new_stream", 3) not in cuda.log
    cuda.log.clear()
    sync = manager.create_stream_work(async_op=False)
    with sync:
        pass
    assert cuda.log == [("wait_stream", "current", "current"), ("enter", "current"), ("exit", "current"),
                        ("record", "current"), "event.wait"]
    assert sync.query() is True
