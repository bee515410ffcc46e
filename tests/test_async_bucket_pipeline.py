"""AsyncBucketPipeline: the order of a bucket's completion behind an asynchronous gather, the optional host wait and
where a failing step ends up - the behaviours of the reference's tests/test_async_bucket_pipeline.py:61-160, with
stand-ins for the gather work, the completion manager and the bucket's future (no GPU)."""
import pytest

from lowbit_comm_amd.communication import AsyncBucketPipeline, GatheredPayloads


class Journal(list):
    def note(self, *entry):
        self.append(entry if len(entry) > 1 else entry[0])


class BucketFuture:
    def __init__(self):
        self.value = self.error = None

    def set_result(self, value):
        self.value = value

    def set_exception(self, error):
        self.error = error


class ResultOnlyFuture:
    def __init__(self):
        self.value = None

    def set_result(self, value):
        self.value = value


class GatherWork:
    """An asynchronous gather of two ranks whose own future fires as soon as somebody chains to it."""

    def __init__(self, journal, with_future=True):
        self.journal = journal
        if with_future:
            self.get_future = self._future

    def _future(self):
        self.journal.note("get_future")
        work = self

        class Inner:
            def then(self, callback):
                work.journal.note("then")
                return callback(self)

        return Inner()

    def wait(self):
        self.journal.note("gather_wait")
        return GatheredPayloads(payloads=["from rank 0", "from rank 1"], world_size=2)


class Completions:
    def __init__(self, journal, can_block_host=True):
        self.journal, self.can_block_host = journal, can_block_host

    def record_for(self, tensor):
        self.journal.note("record", tensor)
        journal = self.journal

        class Done:
            def wait(self):
                journal.note("device_wait")

        if self.can_block_host:
            Done.synchronize = lambda self: journal.note("host_wait")
        return Done()


def pipeline(journal, future, *, work=None, decode=None, **options):
    return AsyncBucketPipeline(
        gather_work=work or GatherWork(journal), future=future,
        dequantize_reduce=decode or (lambda gathered: journal.note("decode", tuple(gathered.payloads)) or "reduced"),
        update_feedback=lambda restored: journal.note("feedback", restored),
        advance_policy=lambda: journal.note("advance"),
        completion_manager=options.pop("completions", Completions(journal)), **options)


def test_steps_run_in_order_behind_the_gathers_own_future():
    journal, future = Journal(), BucketFuture()
    assert pipeline(journal, future).run() is future
    assert journal == ["get_future", "then", "gather_wait", ("decode", ("from rank 0", "from rank 1")), ("feedback", "reduced"),
                       "advance", ("record", "reduced"), "device_wait", "host_wait"]
    assert future.value == "reduced" and future.error is None


def test_a_work_without_a_future_completes_at_once():
    journal, future = Journal(), BucketFuture()
    pipeline(journal, future, work=GatherWork(journal, with_future=False)).run()
    assert journal[0] == "gather_wait" and future.value == "reduced"


def test_the_host_wait_can_be_switched_off_and_is_skipped_when_the_completion_has_none():
    journal, future = Journal(), BucketFuture()
    pipeline(journal, future, synchronize_completion=False).run()
    assert "device_wait" in journal and "host_wait" not in journal and future.value == "reduced"
    journal, future = Journal(), BucketFuture()
    pipeline(journal, future, completions=Completions(journal, can_block_host=False)).run()
    assert journal[-1] == "device_wait" and future.value == "reduced"


def test_a_failing_step_resolves_the_future_with_the_exception_and_skips_the_rest():
    def broken(gathered):
        raise RuntimeError("decode failed")

    journal, future = Journal(), BucketFuture()
    assert pipeline(journal, future, decode=broken).run() is future
    assert isinstance(future.error, RuntimeError) and str(future.error) == "decode failed"
    assert future.value is None
    assert not any(entry in ("advance", "device_wait", "host_wait") for entry in journal)


def test_a_future_that_cannot_carry_an_exception_lets_it_through():
    def broken(gathered):
        raise RuntimeError("decode failed")

    journal, future = Journal(), ResultOnlyFuture()
    with pytest.raises(RuntimeError, match="decode failed"):
        pipeline(journal, future, decode=broken).run()
    assert future.value is None


def test_the_default_completion_manager_is_made_on_demand():
    # no manager given: the pipeline brings the event-based one (it is only asked for a completion when a bucket finishes)
    made = AsyncBucketPipeline(gather_work=GatherWork(Journal()), future=BucketFuture(), dequantize_reduce=lambda g: g,
                               update_feedback=lambda r: None, advance_policy=lambda: None)
    assert type(made._completions).__name__ == "EventCompletionManager"
