"""AsyncShardPipeline: the order of exchange wait, shard reduce, feedback, policy, device ordering, workspace
hand-back and future completion, with and without a future to chain on, and on failure.  Behaviours follow the
reference's tests (tests/test_async_shard_pipeline.py:73-241).  CPU only."""
import pytest

from lowbit_comm_amd.communication import AsyncShardPipeline
from lowbit_comm_amd.shard import ReducedShard


class Outer:
    def __init__(self):
        self.result = None
        self.exception = None

    def set_result(self, value):
        self.result = value

    def set_exception(self, error):
        self.exception = error


class Chained:
    def __init__(self, log):
        self.log = log

    def then(self, callback):
        self.log.append("then")
        return callback(self)


class Exchange:
    def __init__(self, log, with_future=True):
        self.log = log
        if not with_future:
            self.get_future = None

    def get_future(self):
        self.log.append("get_future")
        return Chained(self.log)

    def wait(self):
        self.log.append("wait")
        return ["from-rank-0", "from-rank-1"]


class Ordered:
    def __init__(self, log):
        self.log = log

    def wait(self):
        self.log.append("ordered.wait")

    def synchronize(self):
        self.log.append("ordered.synchronize")


class Completions:
    def __init__(self, log):
        self.log = log

    def record_for(self, value):
        self.log.append(("record_for", value))
        return Ordered(self.log)


class Lease:
    buffer = "leased-buffer"

    def __init__(self, log):
        self.log = log

    def release(self, *, completion):
        self.log.append(("release", completion))


def shard(value):
    return ReducedShard(shard=value, shard_index=0, shard_numel=1, original_shape=(2,), original_numel=2, world_size=2,
                        reduce="mean", dtype="float16", metadata={"kept": 1})


def pipeline(log, outer=None, **changes):
    arguments = dict(communication_work=Exchange(log), future=outer or Outer(),
                     reduce_shard=lambda received: log.append(("reduce", received)) or shard("reduced"),
                     update_feedback=lambda s: log.append(("feedback", s.shard)),
                     advance_policy=lambda: log.append("advance"), completion_manager=Completions(log))
    arguments.update(changes)
    return AsyncShardPipeline(**arguments)


def test_steps_run_in_order_behind_the_exchanges_future():
    log, outer = [], Outer()
    work = pipeline(log, outer)
    assert work.run() is work
    assert log == ["get_future", "then", "wait", ("reduce", ["from-rank-0", "from-rank-1"]), ("feedback", "reduced"),
                   "advance", ("record_for", "reduced"), "ordered.wait"]
    assert work.query() is True and work.wait() is outer.result and work.get_future() is outer
    assert outer.result.shard == "reduced"
    assert outer.result.metadata["async_completion"] is True and outer.result.metadata["kept"] == 1


def test_an_exchange_without_a_future_completes_at_once():
    log = []
    work = pipeline(log, communication_work=Exchange(log, with_future=False)).run()
    assert log[0] == "wait" and work.wait().shard == "reduced"


def test_host_side_wait_is_opt_in_and_comes_last():
    log = []
    pipeline(log, synchronize_completion=True).run()
    assert log[-3:] == [("record_for", "reduced"), "ordered.wait", "ordered.synchronize"]
    log = []
    pipeline(log).run()
    assert "ordered.synchronize" not in log


def test_workspaces_go_back_after_the_result_is_ordered_and_resources_are_only_kept():
    log = []
    kept = object()
    work = pipeline(log, workspace_leases=(Lease(log), Lease(log)), resources=(kept,)).run()
    assert log[-4][0] == "record_for" and log[-3] == "ordered.wait"
    assert [entry[0] for entry in log[-2:]] == ["release", "release"]
    assert log[-1][1] is log[-2][1]                           # both leases get the same completion
    assert work.resources == (kept,)


def test_a_failing_callback_is_delivered_through_the_future_and_still_returns_the_workspaces():
    log, outer = [], Outer()

    def explode(received):
        raise RuntimeError("boom")

    work = pipeline(log, outer, reduce_shard=explode, workspace_leases=(Lease(log),)).run()
    assert isinstance(outer.exception, RuntimeError) and str(outer.exception) == "boom"
    assert log[-3] == ("record_for", Lease.buffer) and log[-2] == "ordered.wait" and log[-1][0] == "release"
    assert work.query() is True
    with pytest.raises(RuntimeError, match="boom"):
        work.wait()


def test_a_future_without_set_exception_lets_the_failure_propagate():
    class ResultOnly:
        result = None

        def set_result(self, value):
            self.result = value

    def explode(received):
        raise ValueError("no channel")

    log = []
    with pytest.raises(ValueError, match="no channel"):
        pipeline(log, ResultOnly(), reduce_shard=explode).run()


def test_wait_before_completion_and_then_without_support_are_errors():
    class Never:
        def get_future(self):
            class Pending:
                def then(self, callback):
                    return None
            return Pending()

        def wait(self):
            raise AssertionError("not reached")

    work = pipeline([], communication_work=Never()).run()
    assert work.query() is False
    with pytest.raises(RuntimeError, match="not complete"):
        work.wait()
    with pytest.raises(AttributeError, match="does not support then"):
        work.then(lambda f: None)


def test_real_torch_future_chains():
    import torch

    log = []
    outer = torch.futures.Future()
    work = pipeline(log, outer).run()
    seen = []
    work.then(lambda f: seen.append(f.value().shard))
    assert work.query() is True and work.wait().shard == "reduced" and seen == ["reduced"]
