"""Stream-ordered completion for compressed collectives on HIP streams.

``HipStreamWork`` runs a body of enqueues on a communication stream that is ordered after the caller's current
stream, and records an event when the body ends; ``HipCompletionManager`` creates it, records completions for
tensors and builds result-bearing :class:`~lowbit_comm_amd.work.CompletionWork` objects.  Counterparts in the
reference: ``CudaStreamWork`` and ``CudaCompletionManager`` (``ccdl_comm/communication/cuda_completion.py:69-260``)
and the native ``CompressedWork`` (``ccdl_comm/csrc/executor/compressed_work.cpp``), whose wait-once and
stream-wait behaviour lives in ``CompletionWork`` here.  Every stream has the default priority.
"""
from __future__ import annotations

from typing import Any, Callable, Sequence

from lowbit_comm_amd.execution_info import ExecutionCounters, ExecutionInfo
from lowbit_comm_amd.hip.workspace import EventCompletionManager, NoopCompletion
from lowbit_comm_amd.work import CompletionWork, ImmediateWork, python_fallback_info

_COMMUNICATION_STREAMS: dict[int, Any] = {}


def communication_stream(cuda: Any) -> Any:
    """One side stream per device, created on first use."""
    device = int(cuda.current_device())
    stream = _COMMUNICATION_STREAMS.get(device)
    if stream is None:
        stream = _COMMUNICATION_STREAMS[device] = cuda.Stream(device)
    return stream


class HipStreamWork:
    """``with work: <enqueue>``: the body runs on ``work.stream`` (the communication stream when ``async_op``, else
    the current stream), which first waits for everything already enqueued on the current stream.  Leaving the
    block records ``work.event``; a synchronous work then orders the current stream after it straight away.
    ``wait()`` waits for the optional transport ``handle`` and, for asynchronous work, orders the caller's current
    stream after the event (a device-side wait: the host does not block)."""

    def __init__(self, *, cuda: Any, async_op: bool = False, handle: Any | None = None) -> None:
        self.async_op = bool(async_op)
        self.handle = handle
        self._cuda = cuda
        self.stream = communication_stream(cuda) if self.async_op else cuda.current_stream()
        self._guard = cuda.stream(self.stream)
        self.event = None

    def __enter__(self) -> "HipStreamWork":
        self.stream.wait_stream(self._cuda.current_stream())
        self._guard.__enter__()
        return self

    def __exit__(self, exc_type: Any, exc_value: Any, traceback: Any) -> None:
        self._guard.__exit__(exc_type, exc_value, traceback)
        self.event = self._cuda.Event()
        self.event.record(self.stream)
        if not self.async_op:
            self.event.wait()

    def wait(self) -> None:
        wait = getattr(self.handle, "wait", None)
        if callable(wait):
            wait()
        if self.async_op and self.event is not None:
            self.event.wait()

    def wait_stream(self, stream: Any) -> None:
        if self.event is not None:
            stream.wait_event(self.event)

    def synchronize(self) -> None:
        if self.event is not None:
            self.event.synchronize()

    def query(self) -> bool:
        if not self.async_op:
            return True
        return self.event is not None and bool(self.event.query())


class HipCompletionManager(EventCompletionManager):
    """``record_for`` (inherited), ``create_stream_work`` and ``create_work``; ``torch_provider`` exists so host-only
    tests can inject a stand-in for ``torch``."""

    def __init__(self, torch_provider: Callable[[], Any] | None = None) -> None:
        self._torch_provider = torch_provider

    def _cuda(self) -> Any | None:
        try:
            if self._torch_provider is not None:
                torch = self._torch_provider()
            else:
                import torch
        except ImportError:
            return None
        cuda = getattr(torch, "cuda", None)
        available = getattr(cuda, "is_available", None)
        if cuda is None or not callable(available) or not available():
            return None
        return cuda

    def create_stream_work(self, *, async_op: bool = False, handle: Any | None = None) -> Any:
        cuda = self._cuda()
        if cuda is None or any(not hasattr(cuda, name) for name in ("current_device", "current_stream", "stream", "Event")):
            return NoopCompletion()
        return HipStreamWork(cuda=cuda, async_op=async_op, handle=handle)

    def create_work(self, *, result: Any, handle: Any | None = None, complete: Callable[[], Any] | None = None,
                    completion: Any | None = None, resources: Sequence[Any] = (),
                    execution_info: ExecutionInfo | None = None,
                    execution_counters: ExecutionCounters | None = None) -> Any:
        """A result-bearing work object; needs no GPU (every part is optional)."""
        if handle is None and complete is None and completion is None and not resources:
            return ImmediateWork(result, execution_info=execution_info, execution_counters=execution_counters)
        return CompletionWork(result, handle=handle, complete=complete, completion=completion, resources=resources,
                              execution_info=python_fallback_info(execution_info),
                              execution_counters=execution_counters)
