"""Host logic of the quantized ring: the compiled schedule (properties the reference states in
tests/cuda/test_topology_executors.py:622-714 and the oracle's message-passing simulation), the executor's call
order and ownership rules (:716-840, 1113-1300).  CPU only."""
import threading

import numpy as np
import pytest

from lowbit_comm_amd.hip.chunk_plan import ChunkRange, compile_chunk_plan
from lowbit_comm_amd.hip.ring import (
    JoinedCompletion,
    PipelinedRingExecutor,
    PipelinedRingSchedule,
    RingAllGatherStep,
    RingReduceScatterStep,
    compile_pipelined_ring_schedule,
)
from oracle import ring_np


@pytest.mark.parametrize("world", [1, 2, 3, 5, 8])
def test_one_step_per_remote_chunk_with_the_stated_owners(world):
    plan = compile_chunk_plan(original_numel=world * 7 + 1, world_size=world)
    for rank in range(world):
        schedule = compile_pipelined_ring_schedule(chunk_plan=plan, rank=rank)
        assert schedule.rank == rank and schedule.chunk_plan is plan
        assert schedule.local_chunk == plan.chunk_for_rank(rank)
        assert [s.step_index for s in schedule.steps] == list(range(world - 1))
        assert [s.step_index for s in schedule.gather_steps] == list(range(world - 1))
        for s in schedule.steps + schedule.gather_steps:
            assert s.send_peer == (rank + 1) % world and s.recv_peer == (rank - 1) % world
            assert s.send_chunk == plan.chunk_for_rank(s.send_chunk_owner)
            assert s.recv_chunk == plan.chunk_for_rank(s.recv_chunk_owner)
        assert [s.send_chunk_owner for s in schedule.steps] == [(rank - i - 1) % world for i in range(world - 1)]
        assert [s.recv_chunk_owner for s in schedule.steps] == [(rank - i - 2) % world for i in range(world - 1)]
        assert [s.send_chunk_owner for s in schedule.gather_steps] == [(rank - i) % world for i in range(world - 1)]
        assert [s.recv_chunk_owner for s in schedule.gather_steps] == [(rank - i - 1) % world for i in range(world - 1)]
        if world > 1:
            assert schedule.steps[-1].recv_chunk_owner == rank
            assert {s.recv_chunk_owner for s in schedule.steps} == set(range(world)) - {(rank - 1) % world}


@pytest.mark.parametrize("world", [2, 3, 5, 8])
def test_provenance_and_restoration_by_simulating_the_messages(world):
    plan = compile_chunk_plan(original_numel=world * 5, world_size=world)
    schedules = [compile_pipelined_ring_schedule(chunk_plan=plan, rank=r) for r in range(world)]
    held = [{owner: (rank,) for owner in range(world)} for rank in range(world)]
    for i in range(world - 1):
        in_flight = {(r, s.steps[i].send_peer): held[r][s.steps[i].send_chunk_owner] for r, s in enumerate(schedules)}
        for r, s in enumerate(schedules):
            step = s.steps[i]
            arriving = in_flight[(step.recv_peer, r)]
            assert step.received_contributors == arriving
            assert not set(arriving) & set(held[r][step.recv_chunk_owner])
            held[r][step.recv_chunk_owner] = arriving + held[r][step.recv_chunk_owner]
    assert all(set(held[r][r]) == set(range(world)) for r in range(world))
    complete = [{r} for r in range(world)]
    for i in range(world - 1):
        in_flight = {(r, s.gather_steps[i].send_peer): s.gather_steps[i].send_chunk_owner
                     for r, s in enumerate(schedules)}
        for r, s in enumerate(schedules):
            step = s.gather_steps[i]
            assert in_flight[(step.recv_peer, r)] == step.recv_chunk_owner
            assert step.send_chunk_owner in complete[r]           # only complete chunks are handed on
            complete[r].add(step.recv_chunk_owner)
    assert all(c == set(range(world)) for c in complete)


@pytest.mark.parametrize("world", [2, 3, 8])
def test_compiled_schedule_agrees_with_the_oracles_message_passing(world):
    n = world * 16 + 3
    trace = []
    ring_np.ring_all_reduce([np.zeros(n, np.float32)] * world, "fp32", 16, trace=trace)
    plan = compile_chunk_plan(original_numel=n, world_size=world)
    for rank in range(world):
        schedule = compile_pipelined_ring_schedule(chunk_plan=plan, rank=rank)
        mine = [t for t in trace if t[2] == rank]
        reduce = [(t[1], t[3], t[4], t[5]) for t in mine if t[0] == "reduce"]
        gather = [(t[1], t[3], t[4], t[5]) for t in mine if t[0] == "gather"]
        assert reduce == [(s.step_index, s.send_chunk_owner, s.recv_peer, s.recv_chunk_owner) for s in schedule.steps]
        assert gather == [(s.step_index, s.send_chunk_owner, s.recv_peer, s.recv_chunk_owner)
                          for s in schedule.gather_steps]


def test_schedule_metadata_is_validated_and_immutable():
    plan = compile_chunk_plan(original_numel=15, world_size=3)
    schedule = compile_pipelined_ring_schedule(chunk_plan=plan, rank=2)
    with pytest.raises(Exception):
        schedule.rank = 0
    with pytest.raises(ValueError, match="deterministic ring schedule"):
        PipelinedRingSchedule(chunk_plan=plan, rank=1, steps=schedule.steps, gather_steps=schedule.gather_steps)
    with pytest.raises(TypeError, match="chunk_plan must be a ChunkPlan"):
        compile_pipelined_ring_schedule(chunk_plan=object(), rank=0)
    with pytest.raises(ValueError, match=r"rank must be in \[0, 3\)"):
        compile_pipelined_ring_schedule(chunk_plan=plan, rank=3)
    with pytest.raises(TypeError, match="rank must be an integer"):
        compile_pipelined_ring_schedule(chunk_plan=plan, rank=True)
    chunk = ChunkRange(0, 5)
    good = dict(step_index=1, send_peer=0, recv_peer=1, send_chunk_owner=0, recv_chunk_owner=1,
                received_contributors=(0, 1), send_chunk=chunk, recv_chunk=chunk)
    RingReduceScatterStep(**good)
    for change, error, text in (({"received_contributors": (0,)}, ValueError, "step_index \\+ 1"),
                                ({"received_contributors": (1, 1)}, ValueError, "duplicates"),
                                ({"received_contributors": [0, 1]}, TypeError, "must be a tuple"),
                                ({"step_index": 0, "received_contributors": ()}, ValueError, "must not be empty"),
                                ({"send_peer": -1}, ValueError, "send_peer must be >= 0"),
                                ({"recv_chunk": (0, 5)}, TypeError, "recv_chunk must be a ChunkRange")):
        with pytest.raises(error, match=text):
            RingReduceScatterStep(**{**good, **change})
    with pytest.raises(TypeError, match="send_chunk must be a ChunkRange"):
        RingAllGatherStep(step_index=0, send_peer=0, recv_peer=0, send_chunk_owner=0, recv_chunk_owner=0,
                          send_chunk=None, recv_chunk=chunk)


# --------------------------------------------------------------------------- #
# executor
# --------------------------------------------------------------------------- #
class Endpoint:
    def __init__(self, ready=True):
        self.ready = ready
        self.stream_waits = []

    def query(self):
        return self.ready

    def wait(self):
        return None

    def wait_stream(self, stream):
        self.stream_waits.append(stream)


class Handle:
    def __init__(self):
        self.done = True

    def is_completed(self):
        return self.done


class Runtime:
    def __init__(self, fail_at=None, handle_factory=Handle):
        self.calls = []
        self.context = Endpoint()
        self.completion = Endpoint()
        self.handles = []
        self.recorded_dependencies = None
        self.fail_at = fail_at
        self.handle_factory = handle_factory

    def _maybe_fail(self, name):
        if self.fail_at == name:
            raise RuntimeError(f"{name} failed")

    def create_submission_context(self, tensor):
        self.calls.append(("create_submission_context", tensor))
        return self.context

    def wait_for_producer(self, tensor, *, context):
        assert context is self.context
        self.calls.append(("producer_wait", tensor))

    def quant_pack(self, tensor, chunk, workspace, *, context):
        self.calls.append(("quant_pack", chunk, workspace))
        self._maybe_fail("quant_pack")
        return ("payload", chunk)

    def send_recv(self, payload, *, send_peer, recv_peer, recv_chunk, workspace, context):
        self.calls.append(("send_recv", send_peer, recv_peer, recv_chunk, workspace))
        handle = self.handle_factory()
        self.handles.append(handle)
        return ("received", recv_chunk), handle

    def fused_reduce(self, tensor, received, chunk, contributors, workspace, *, context, dependency):
        assert dependency is self.handles[-1]
        self.calls.append(("fused_reduce", chunk, contributors, workspace))
        self._maybe_fail("fused_reduce")
        return None

    def apply_broadcast(self, tensor, received, chunk, workspace, *, context, dependency):
        assert dependency is self.handles[-1]
        self.calls.append(("apply_broadcast", chunk, workspace))
        return None

    def record_completion(self, *, context, dependencies):
        self.calls.append("record_completion")
        self._maybe_fail("record_completion")
        self.recorded_dependencies = dependencies
        return self.completion


class Session:
    def __init__(self, with_abort=True):
        self.released_with = []
        self.aborts = 0
        if not with_abort:
            self.abort = None

    def release(self, *, completion):
        self.released_with.append(completion)

    def abort(self):
        self.aborts += 1


class Work:
    def __init__(self, result, completion, resources):
        self.result, self.completion, self.resources = result, completion, resources


class Works:
    def create_work(self, *, result, completion, resources):
        return Work(result, completion, resources)


def make(world=3, rank=1, runtime=None, session=None):
    plan = compile_chunk_plan(original_numel=15, world_size=world)
    schedule = compile_pipelined_ring_schedule(chunk_plan=plan, rank=rank)
    runtime = runtime or Runtime()
    session = session or Session()
    executor = PipelinedRingExecutor(schedule=schedule, runtime=runtime, workspace_session_factory=lambda t: session,
                                     completion_manager=Works())
    return schedule, runtime, session, executor


def test_executor_submits_every_step_in_order_and_hands_ownership_to_the_work():
    schedule, runtime, session, executor = make()
    tensor = object()
    work = executor.run(tensor)
    expected = [("create_submission_context", tensor), ("producer_wait", tensor)]
    for step in schedule.steps:
        expected += [("quant_pack", step.send_chunk, session),
                     ("send_recv", step.send_peer, step.recv_peer, step.recv_chunk, session),
                     ("fused_reduce", step.recv_chunk, step.received_contributors, session)]
    for step in schedule.gather_steps:
        expected += [("quant_pack", step.send_chunk, session),
                     ("send_recv", step.send_peer, step.recv_peer, step.recv_chunk, session),
                     ("apply_broadcast", step.recv_chunk, session)]
    assert runtime.calls == expected + ["record_completion"]
    assert work.result is tensor
    assert isinstance(work.completion, JoinedCompletion)
    assert work.completion.context is runtime.context and work.completion.runtime_completion is runtime.completion
    assert session in work.resources and all(h in work.resources for h in runtime.handles)
    assert all(h in runtime.recorded_dependencies for h in runtime.handles)
    assert session.released_with == [work.completion] and session.aborts == 0
    assert executor.pending_submission_count == 0
    assert [len(s.received_contributors) for s in schedule.steps] == [1, 2]


def test_executor_rejects_wrong_collaborators_and_blocking_only_p2p_handles():
    plan = compile_chunk_plan(original_numel=15, world_size=3)
    schedule = compile_pipelined_ring_schedule(chunk_plan=plan, rank=0)
    with pytest.raises(TypeError, match="schedule must be a PipelinedRingSchedule"):
        PipelinedRingExecutor(schedule=object(), runtime=Runtime(), workspace_session_factory=lambda t: None,
                              completion_manager=Works())
    with pytest.raises(TypeError, match="workspace_session_factory must be callable"):
        PipelinedRingExecutor(schedule=schedule, runtime=Runtime(), workspace_session_factory=None,
                              completion_manager=Works())

    class WaitOnly:
        def wait(self):
            return None

    _, runtime, session, executor = make(runtime=Runtime(handle_factory=WaitOnly))
    with pytest.raises(TypeError, match="nonblocking query\\(\\) or is_completed\\(\\)"):
        executor.run(object())
    assert session.released_with == [] and executor.pending_submission_count == 1
    executor.reap_pending()                                   # the recorded completion is ready: abort once
    assert session.aborts == 1 and executor.pending_submission_count == 0

    class NoWaitStream:
        def query(self):
            return True

        def wait(self):
            return None

    bad_context = Runtime()
    bad_context.context = NoWaitStream()
    _, _, _, executor = make(runtime=bad_context)
    with pytest.raises(TypeError, match="submission context must provide wait_stream"):
        executor.run(object())


def test_a_failing_step_aborts_the_session_once_after_the_device_work_has_drained():
    runtime = Runtime(fail_at="fused_reduce")
    runtime.completion.ready = False
    _, _, session, executor = make(runtime=runtime)
    with pytest.raises(RuntimeError, match="fused_reduce failed"):
        executor.run(object())
    assert "record_completion" in runtime.calls               # something to wait for before buffers go back
    assert session.aborts == 0 and executor.pending_submission_count == 1
    executor.reap_pending()
    assert session.aborts == 0                                # device work still in flight
    runtime.completion.ready = True
    executor.reap_pending()
    assert session.aborts == 1 and session.released_with == [] and executor.pending_submission_count == 0
    executor.reap_pending()
    assert session.aborts == 1


def test_a_failing_record_is_not_retried_and_a_session_without_abort_is_released():
    runtime = Runtime(fail_at="record_completion")
    session = Session(with_abort=False)
    _, _, _, executor = make(runtime=runtime, session=session)
    with pytest.raises(RuntimeError, match="record_completion failed"):
        executor.run(object())
    assert runtime.calls.count("record_completion") == 1
    assert executor.pending_submission_count == 1
    executor.reap_pending()                                   # falls back to the context's readiness
    assert session.released_with == [runtime.context] and executor.pending_submission_count == 0


def test_workspace_factory_failure_transfers_no_ownership():
    plan = compile_chunk_plan(original_numel=15, world_size=3)
    schedule = compile_pipelined_ring_schedule(chunk_plan=plan, rank=0)

    def factory(tensor):
        raise MemoryError("no workspace")

    executor = PipelinedRingExecutor(schedule=schedule, runtime=Runtime(), workspace_session_factory=factory,
                                     completion_manager=Works())
    with pytest.raises(MemoryError):
        executor.run(object())
    assert executor.pending_submission_count == 0


def test_concurrent_submission_and_reaping_during_a_submission_are_rejected():
    entered, leave = threading.Event(), threading.Event()

    class Slow(Runtime):
        def wait_for_producer(self, tensor, *, context):
            entered.set()
            assert leave.wait(10)

    _, _, _, executor = make(runtime=Slow())
    errors = []
    thread = threading.Thread(target=lambda: executor.run(object()))
    thread.start()
    assert entered.wait(10)
    for call, text in ((lambda: executor.run(object()), "concurrent run"), (executor.reap_pending, "cannot reap")):
        try:
            call()
        except RuntimeError as error:
            errors.append(str(error))
            assert text in str(error)
    leave.set()
    thread.join(10)
    assert len(errors) == 2


def test_joined_completion_needs_both_endpoints_and_orders_a_stream_after_both():
    a, b = Endpoint(), Endpoint(ready=False)
    joined = JoinedCompletion(a, b)
    assert joined.query() is False and joined.is_completed() is False
    b.ready = True
    assert joined.query() is True
    joined.wait_stream("s")
    assert a.stream_waits == ["s"] and b.stream_waits == ["s"]
    with pytest.raises(TypeError, match="runtime completion must provide nonblocking"):
        JoinedCompletion(a, object())


def test_runtime_rejects_policies_the_ring_step_kernel_does_not_serve():
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.hip.ring import HipPipelinedRingRuntime

    def exchange(*args, **kwargs):
        raise AssertionError("not reached")

    ok = dict(dtype="fp32", world_size=4, rank=0, exchange=exchange)
    HipPipelinedRingRuntime(config=CompressionConfig(), **ok)
    with pytest.raises(ValueError, match="requires topk=0"):
        HipPipelinedRingRuntime(config=CompressionConfig(topk=2), **ok)
    with pytest.raises(ValueError, match="unsupported dtype"):
        HipPipelinedRingRuntime(config=CompressionConfig(), **{**ok, "dtype": "fp64"})
    with pytest.raises(ValueError, match=r"rank must be in \[0, 4\)"):
        HipPipelinedRingRuntime(config=CompressionConfig(), **{**ok, "rank": 4})
    with pytest.raises(TypeError, match="exchange must be callable"):
        HipPipelinedRingRuntime(config=CompressionConfig(), **{**ok, "exchange": None})
