"""Scheduling of the bucket pipeline without a GPU: which stages share a launch, in which order the exchanges are
called, when futures complete, what a flush issues.  The plans and the merged launch are replaced by recorders; the
kernels behind them are covered by the GPU tests (tests/test_bucket_pipeline.py).

What the reference fixes here is the order of one bucket's steps - quantize, exchange, reduce, (requantize, gather,
decode), complete (ccdl_comm/communication/reduce_scatter_transport.py:262-347,
ccdl_comm/communication/async_shard_pipeline.py:93-110) - which the pipeline keeps per bucket while it overlaps the
steps of neighbouring buckets."""
import threading

import pytest
import torch

from lowbit_comm_amd import CompressionConfig
from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
from lowbit_comm_amd.hip.bucket_pipeline import BucketPipeline

CFG = CompressionConfig()


class FakeLaunch:
    def __init__(self, log, what, works=True):
        self.log, self.what, self.works = log, what, works

    def __call__(self, stream=None):
        self.log.append(self.what)
        return self.works


class FakePlan:
    """Stands where ReduceScatterPlan stands: hands out recorders instead of bound kernels."""

    made = 0

    def __init__(self, numel, dtype, *, world_size, rank, config, device, shape=None, log=None):
        FakePlan.made += 1
        self.tag = FakePlan.made
        self.numel, self.dtype, self.reduced_dtype, self.world_size, self.rank = numel, dtype, dtype, world_size, rank
        self.shape = tuple(shape) if shape is not None else (numel,)
        self.send = ("send", self.tag)
        self.received = ("received", self.tag)
        self.gathered = ("gathered", self.tag)
        self.my_row = ("row", self.gathered, rank)
        self.log = log
        self.chunks = type("Chunks", (), {"shard_numel": -(-numel // world_size)})()
        self._launches = {}

    def _order_after_previous_use(self):
        pass

    def payload(self, rows, index):
        return ("row", rows, index)

    def _launch(self, what):
        if what not in self._launches:
            self._launches[what] = FakeLaunch(self.log, what)
        return self._launches[what]

    def bound_quantize(self, tensor, *, residual=None, new_residual=None):
        return self._launch(("Q", tensor.bucket_id, residual is not None))

    def bound_reduce_requantize(self, received=None, *, op="sum"):
        return self._launch(("RQ", self.tag, op))

    def bound_reduce(self, received=None, *, op="sum", out=None):
        return self._launch(("R", self.tag, op))

    def bound_decode(self, target, gathered=None, *, remember=True):
        return self._launch(("D", self.tag))

    def reduced_shard(self, target, *, op, fused=True, caller_owned=False):
        return ("shard", self.tag, op)


class Tensor(torch.Tensor):
    pass


def bucket_tensor(bucket_id, numel=640):
    t = torch.zeros(numel).as_subclass(Tensor)
    t.bucket_id = bucket_id
    return t


def make_pipeline(log, *, full=True, merge_works=True, **kwargs):
    def merge(quant, reduce, decode):
        parts = tuple(p.what for p in (quant, reduce, decode) if p is not None)
        return FakeLaunch(log, ("MERGED",) + parts, works=merge_works)

    def all_to_all(received, send):
        log.append(("a2a", received, send))

    def all_gather(gathered, mine):
        log.append(("ag", gathered, mine))

    FakePlan.made = 0
    return BucketPipeline(world_size=8, rank=0, all_to_all=all_to_all, all_gather=all_gather if full else None,
                          plan_factory=lambda *a, **k: FakePlan(*a, log=log, **k), merge_stages=merge,
                          future_factory=torch.futures.Future, **kwargs)


def test_full_plan_one_launch_per_bucket_and_per_bucket_order_kept():
    log = []
    pipe = make_pipeline(log)
    tensors = [bucket_tensor(k) for k in range(4)]
    futures = [pipe.submit(t, config=CFG, op="mean") for t in tensors]
    # bucket 0: alone; bucket 1: with the reduce of 0; buckets 2, 3: all three stages
    launches = [entry for entry in log if entry[0] in ("Q", "MERGED")]
    assert launches[0] == ("Q", 0, False)
    assert launches[1] == ("MERGED", ("Q", 1, False), ("RQ", 1, "mean"))
    assert launches[2] == ("MERGED", ("Q", 2, False), ("RQ", 2, "mean"), ("D", 1))
    assert launches[3] == ("MERGED", ("Q", 3, False), ("RQ", 3, "mean"), ("D", 2))
    assert [f.done() for f in futures] == [True, True, False, False]
    assert pipe.pending == 2
    pipe.flush()
    assert [f.done() for f in futures] == [True] * 4 and pipe.pending == 0
    tail = [entry for entry in log if entry[0] in ("Q", "MERGED", "D")][4:]
    assert tail == [("MERGED", ("RQ", 1, "mean"), ("D", 3)), ("D", 1)]       # plan 1 again: three plans per shape
    # per bucket: launch with its quantize < its all-to-all < launch with its reduce < its all-gather < launch with
    # its decode; bucket k uses plan (k mod 3) + 1
    for k in range(4):
        plan = k % 3 + 1
        position = {}
        for at, entry in enumerate(log):
            flat = entry if entry[0] != "MERGED" else entry[1:]
            names = [flat] if entry[0] != "MERGED" else list(flat)
            for name in names:
                if name == ("Q", k, False):
                    position["Q"] = at
                if name == ("a2a", ("received", plan), ("send", plan)) and "Q" in position and "a2a" not in position:
                    position["a2a"] = at
                if name == ("RQ", plan, "mean") and "a2a" in position and "RQ" not in position:
                    position["RQ"] = at
                if name[0] == "ag" and name[1] == ("gathered", plan) and "RQ" in position and "ag" not in position:
                    position["ag"] = at
                if name == ("D", plan) and "ag" in position and "D" not in position:
                    position["D"] = at
        assert list(position) == ["Q", "a2a", "RQ", "ag", "D"], (k, position)
    assert pipe.stats["merged_launches"] == 4 and pipe.stats["separate_launches"] == 2 and pipe.stats["buckets"] == 4
    for k, future in enumerate(futures):
        assert future.wait().data_ptr() == tensors[k].data_ptr()          # decoded in place


def test_reduce_scatter_leg_alone_merges_quantize_with_the_previous_reduce():
    log = []
    pipe = make_pipeline(log, full=False)
    futures = [pipe.submit(bucket_tensor(k), config=CFG, op="sum") for k in range(3)]
    launches = [entry for entry in log if entry[0] in ("Q", "R", "MERGED")]
    assert launches == [("Q", 0, False), ("MERGED", ("Q", 1, False), ("R", 1, "sum")), ("MERGED", ("Q", 2, False), ("R", 2, "sum"))]
    assert [f.done() for f in futures] == [True, True, False]
    assert futures[0].wait() == ("shard", 1, "sum") and futures[1].wait() == ("shard", 2, "sum")
    pipe.flush()
    assert futures[2].wait() == ("shard", 1, "sum")                       # two plans per shape: bucket 2 is on plan 1 again
    assert log[-1] == ("R", 1, "sum")
    assert not [entry for entry in log if entry[0] == "ag"]


def test_no_shared_grid_falls_back_to_the_same_stages_in_the_same_order():
    log = []
    pipe = make_pipeline(log, merge_works=False)
    for k in range(3):
        pipe.submit(bucket_tensor(k), config=CFG)
    pipe.flush()
    kernels = [entry for entry in log if entry[0] in ("Q", "RQ", "D")]
    assert kernels == [("Q", 0, False), ("Q", 1, False), ("RQ", 1, "mean"), ("Q", 2, False), ("RQ", 2, "mean"), ("D", 1),
                       ("RQ", 3, "mean"), ("D", 2), ("D", 3)]
    assert pipe.stats["merged_launches"] == 0 and pipe.stats["separate_launches"] == 9


def test_an_exchange_that_returns_work_is_waited_for_right_before_the_launch_that_reads_it():
    log = []

    class Work:
        def __init__(self, name):
            self.name = name

        def wait(self):
            log.append(("wait", self.name))

    pipe = make_pipeline(log)
    pipe.all_to_all = lambda received, send: log.append(("a2a", received)) or Work(("a2a", received))
    pipe.all_gather = lambda gathered, mine: log.append(("ag", gathered)) or Work(("ag", gathered))
    for k in range(3):
        pipe.submit(bucket_tensor(k), config=CFG)
    pipe.flush()
    for name in [("a2a", ("received", p)) for p in (1, 2, 3)] + [("ag", ("gathered", p)) for p in (1, 2, 3)]:
        issued, waited = log.index(name), log.index(("wait", name))
        stage = ("RQ" if name[0] == "a2a" else "D", name[1][1])
        reader = next(at for at, entry in enumerate(log) if at > issued and (
            entry[:2] == stage or (entry[0] == "MERGED" and any(part[:2] == stage for part in entry[1:]))))
        assert issued < waited < reader
        assert not any(entry[0] in ("Q", "RQ", "D", "MERGED") for entry in log[waited + 1:reader])


def test_shapes_of_one_stream_get_their_own_plans_and_the_turn_restarts_after_a_flush():
    log = []
    pipe = make_pipeline(log)
    sizes = [640, 640, 320, 640, 640]
    for _ in range(2):
        for k, size in enumerate(sizes):
            pipe.submit(bucket_tensor(k, size), config=CFG)
        pipe.flush()
    quantized_on = {}
    for entry in log:
        if entry[0] == "a2a":
            quantized_on.setdefault("order", []).append(entry[1][1])
    first, second = quantized_on["order"][:5], quantized_on["order"][5:]
    assert first == second                           # a bucket meets the same plan in the next iteration
    assert len(set(first[:2] + first[3:])) == 3 and first[2] not in first[:2] + first[3:]
    assert FakePlan.made == 6                        # three per shape


def test_error_feedback_residuals_are_kept_per_bucket_and_dropped_by_reset():
    log = []
    pipe = make_pipeline(log, error_feedback=True)
    a, b = bucket_tensor(0), bucket_tensor(1)
    for _ in range(2):
        pipe.submit(a, config=CFG)
        pipe.submit(b, config=CFG)
        pipe.flush()
    assert len(pipe.residuals) == 2
    assert all(r.dtype == torch.float32 and r.numel() == 640 for r in pipe.residuals.values())
    assert [entry for entry in log if entry[0] == "Q"] == [("Q", 0, True), ("Q", 0, True)]
    pipe.reset()
    assert pipe.residuals == {}


def test_residual_store_is_bounded_and_drops_the_least_recently_used():
    log = []
    pipe = make_pipeline(log, error_feedback=True, max_residuals=2)
    a, b, c = bucket_tensor(0), bucket_tensor(1), bucket_tensor(2)
    key = lambda t: (t.data_ptr(), t.numel(), t.dtype)
    pipe.submit(a, config=CFG)
    pipe.submit(b, config=CFG)
    first_a = pipe.residuals[key(a)]
    pipe.submit(a, config=CFG)                       # a is the most recently used now
    pipe.submit(c, config=CFG)                       # ... so b's residual is the one that goes
    pipe.flush()
    assert set(pipe.residuals) == {key(a), key(c)}
    assert pipe.residuals[key(a)] is first_a         # a residual that stays is the same tensor, not a new zero one
    with pytest.raises(ValueError, match="max_entries"):
        make_pipeline(log, error_feedback=True, max_residuals=0)


def test_the_same_memory_again_while_in_flight_finishes_the_earlier_bucket_first():
    log = []
    pipe = make_pipeline(log)
    a, b = bucket_tensor(0), bucket_tensor(1)
    first = pipe.submit(a, config=CFG)
    pipe.submit(b, config=CFG)
    assert not first.done()
    again = pipe.submit(a, config=CFG)               # would be quantized while its earlier result is decoded into it
    assert first.done() and not again.done() and pipe.pending == 1
    decodes = [i for i, entry in enumerate(log) if entry[0] == "D" or (entry[0] == "MERGED" and any(p[0] == "D" for p in entry[1:]))]
    quantizes = [i for i, entry in enumerate(log) if entry == ("Q", 0, False)]
    assert len(quantizes) == 2 and max(decodes) < quantizes[1]    # every earlier decode precedes the second quantize
    view = a[:320]                                    # an overlapping view counts as the same memory
    view.bucket_id = 2
    pipe.submit(view, config=CFG)
    assert again.done()
    pipe.flush()


def test_a_flush_that_raised_is_retried_by_the_next_one():
    log = []
    pipe = make_pipeline(log)
    failures = [RuntimeError("link down")]
    inner = pipe.all_gather

    def flaky_all_gather(gathered, mine):
        if failures:
            raise failures.pop()
        return inner(gathered, mine)

    futures = [pipe.submit(bucket_tensor(k), config=CFG) for k in range(2)]
    pipe.all_gather = flaky_all_gather               # the first exchange of the flush fails
    with pytest.raises(RuntimeError, match="link down"):
        pipe.flush()
    assert pipe.pending == 2 and not any(f.done() for f in futures)
    pipe.flush()                                     # the stages of the failed step go out again, then the rest
    assert pipe.pending == 0 and all(f.done() for f in futures)
    issued = len(log)
    pipe.flush()                                     # nothing is left: nothing is issued
    assert len(log) == issued


def test_empty_buckets_complete_at_once_and_invalid_requests_are_refused():
    log = []
    pipe = make_pipeline(log)
    empty = bucket_tensor(0, 0)
    assert pipe.submit(empty, config=CFG).wait() is empty and log == []
    with pytest.raises(ValueError, match="unsupported reduce-scatter mode"):
        pipe.submit(bucket_tensor(1), config=CFG, op="max")
    with pytest.raises(ValueError, match="out does not match"):
        pipe.submit(bucket_tensor(1), config=CFG, out=torch.zeros(3))
    with pytest.raises(ValueError, match="lanes"):
        BucketPipeline(world_size=8, rank=0, all_to_all=print, lanes=0)
    wide = BucketPipeline(world_size=9, rank=0, all_to_all=print, all_gather=print,
                          plan_factory=lambda *a, **k: FakePlan(*a, log=log, **k))
    with pytest.raises(ValueError, match="at most 8 ranks"):
        wide.submit(bucket_tensor(2), config=CFG)


def test_default_futures_flush_the_pipeline_when_somebody_waits():
    log = []

    def merge(quant, reduce, decode):
        return FakeLaunch(log, "MERGED")

    pipe = BucketPipeline(world_size=8, rank=0, all_to_all=lambda r, s: None, all_gather=lambda g, m: None,
                          plan_factory=lambda *a, **k: FakePlan(*a, log=log, **k), merge_stages=merge)
    futures = [pipe.submit(bucket_tensor(k), config=CFG) for k in range(3)]
    assert not futures[2].done() and pipe.pending == 2
    futures[2].wait()
    assert pipe.pending == 0 and all(f.done() for f in futures)


def test_two_threads_submitting_and_flushing_do_not_corrupt_the_pipeline():
    log = []
    pipe = make_pipeline(log)
    errors = []

    def worker(base):
        try:
            for k in range(200):
                pipe.submit(bucket_tensor(base + k), config=CFG)
                if k % 7 == 0:
                    pipe.flush()
        except Exception as failure:      # noqa: BLE001
            errors.append(failure)

    threads = [threading.Thread(target=worker, args=(1000 * i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    pipe.flush()
    assert not errors and pipe.pending == 0 and pipe.stats["buckets"] == 400
    quantized = [e for entry in log for e in ([entry] if entry[0] == "Q" else entry[1:] if entry[0] == "MERGED" else [])
                 if e[0] == "Q"]
    assert len(quantized) == 400


# ---- the comm hook flushes after the iteration's last bucket ---------------------------------------------------------
class Bucket:
    def __init__(self, tensor, index, last):
        self._tensor, self._index, self._last = tensor, index, last

    def buffer(self):
        return self._tensor

    def index(self):
        return self._index

    def is_last(self):
        return self._last


def test_hook_flushes_a_pipelined_transport_after_the_last_bucket():
    log = []
    pipe = make_pipeline(log)

    def transport(tensor, *, config, op, async_op, dtype, extension_status):
        return pipe.submit(tensor, config=config, op=op)

    transport.pipelined = True
    transport.flush = pipe.flush
    hook = create_ddp_comm_hook(CFG, strategy="reduce_scatter", reduce="mean", reduce_scatter_all_gather=transport,
                                dtype="fp32")
    futures = [hook(None, Bucket(bucket_tensor(k), k, last=(k == 3))) for k in range(4)]
    assert all(f.done() for f in futures) and pipe.pending == 0 and pipe.stats["flushes"] == 1
    # a transport that is not pipelined is never asked to flush
    calls = []

    def plain(tensor, *, config, op, async_op, dtype, extension_status):
        return tensor

    plain.flush = lambda: calls.append("flush")
    hook = create_ddp_comm_hook(CFG, strategy="reduce_scatter", reduce="mean", reduce_scatter_all_gather=plain, dtype="fp32")
    hook(None, Bucket(bucket_tensor(0), 0, last=True))
    assert calls == []


def test_hook_flushes_after_every_bucket_that_cannot_say_whether_it_is_the_last():
    """DistributedDataParallel waits for a hook's futures where a Python override of wait() is not seen: a bucket
    object without is_last() must not leave its future behind in the pipeline."""
    log = []
    pipe = make_pipeline(log)

    def transport(tensor, *, config, op, async_op, dtype, extension_status):
        return pipe.submit(tensor, config=config, op=op)

    transport.pipelined = True
    transport.flush = pipe.flush

    class Anonymous:
        def __init__(self, tensor, index):
            self._tensor, self._index = tensor, index

        def buffer(self):
            return self._tensor

        def index(self):
            return self._index

    hook = create_ddp_comm_hook(CFG, strategy="reduce_scatter", reduce="mean", reduce_scatter_all_gather=transport,
                                dtype="fp32")
    for k in range(3):
        assert hook(None, Anonymous(bucket_tensor(k), k)).done() and pipe.pending == 0
    assert pipe.stats["flushes"] == 3


def test_hook_flushes_when_the_last_bucket_is_too_small_to_compress():
    log = []
    pipe = make_pipeline(log)

    def transport(tensor, *, config, op, async_op, dtype, extension_status):
        return pipe.submit(tensor, config=config, op=op)

    transport.pipelined = True
    transport.flush = pipe.flush
    hook = create_ddp_comm_hook(CFG, strategy="reduce_scatter", reduce="mean", reduce_scatter_all_gather=transport,
                                dtype="fp32", min_compress_numel=100, bypass_all_reduce=lambda t, r: t)
    first = hook(None, Bucket(bucket_tensor(0), 0, last=False))
    assert pipe.pending == 1
    hook(None, Bucket(bucket_tensor(1, 10), 1, last=True))
    assert pipe.pending == 0 and first.done()


# ---- the all-gather form: one payload per bucket, gathered whole, reduced into the bucket ------------------------------
def make_gather_pipeline(log, **kwargs):
    def merge(quant, reduce, decode):
        assert decode is None
        return FakeLaunch(log, ("MERGED",) + tuple(p.what for p in (quant, reduce) if p is not None))

    def whole_gather(received, mine):
        log.append(("gather", received, mine))

    def plan(*a, **k):
        made = FakePlan(*a, log=log, **k)
        made.my_payload = ("payload", made.tag)
        return made

    FakePlan.made = 0
    return BucketPipeline(world_size=8, rank=0, whole_gather=whole_gather, plan_factory=plan, merge_stages=merge,
                          future_factory=torch.futures.Future, **kwargs)


def test_all_gather_form_merges_the_quantize_with_the_previous_buckets_reduce():
    log = []
    pipe = make_gather_pipeline(log)
    tensors = [bucket_tensor(k) for k in range(3)]
    futures = [pipe.submit(t, config=CFG, op="mean") for t in tensors]
    assert log == [
        ("Q", 0, False), ("gather", ("received", 1), ("payload", 1)),
        ("MERGED", ("Q", 1, False), ("R", 1, "mean")), ("gather", ("received", 2), ("payload", 2)),
        ("MERGED", ("Q", 2, False), ("R", 2, "mean")), ("gather", ("received", 1), ("payload", 1)),   # two plans per shape
    ]
    assert [f.done() for f in futures] == [True, True, False] and pipe.pending == 1
    pipe.flush()
    assert log[-1] == ("R", 1, "mean") and futures[2].done() and pipe.pending == 0
    for tensor, future in zip(tensors, futures):
        assert future.wait().data_ptr() == tensor.data_ptr() and future.wait().shape == tensor.shape   # reduced in place


def test_all_gather_form_with_error_feedback_hands_the_buckets_residual_to_the_quantize():
    log = []
    pipe = make_gather_pipeline(log, error_feedback=True)
    first, second = bucket_tensor(0), bucket_tensor(1)
    for _ in range(2):
        pipe.submit(first, config=CFG)
        pipe.submit(second, config=CFG)
        pipe.flush()
    assert [entry for entry in log if entry[0] == "Q"] == [("Q", 0, True), ("Q", 0, True)]
    assert len(pipe.residuals) == 2


def test_the_two_forms_exclude_each_other():
    with pytest.raises(ValueError, match="either all_to_all"):
        BucketPipeline(world_size=2, rank=0)
    with pytest.raises(ValueError, match="either all_to_all"):
        BucketPipeline(world_size=2, rank=0, all_to_all=lambda r, s: None, whole_gather=lambda r, m: None)
    with pytest.raises(ValueError, match="one exchange"):
        BucketPipeline(world_size=2, rank=0, whole_gather=lambda r, m: None, all_gather=lambda g, m: None)
