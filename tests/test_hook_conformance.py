"""Behaviour of ``create_ddp_comm_hook`` and ``DDPBucketProcessor`` under duck-typed stand-ins.

Each case states a contract a caller of the reference's hook relies on
(ccdl_comm/communication/ddp_hook.py:48-369; the scenarios are those its own test-suite walks through in
tests/test_ddp_comm_hook.py and tests/test_ddp_hook_scaffold.py): which callables run, in which order, with
which arguments, and what the returned future holds.  No GPU and no torch tensors are involved.
"""
from __future__ import annotations

import pytest

import lowbit_comm_amd.communication.ddp_hook as hook_module
from lowbit_comm_amd.communication.collectives import CompressedPayload
from lowbit_comm_amd.communication.ddp import DDPBucketProcessor
from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
from lowbit_comm_amd.communication.gather_reduce import GatheredPayloads
from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.exceptions import UnsupportedCollective


class Vec:
    """The least a bucket tensor must offer: shape, dtype, numel, clone, + and /."""

    def __init__(self, *values, dtype=None):
        self.values = tuple(float(v) for v in values)
        self.shape = (len(self.values),)
        self.dtype = dtype

    def numel(self):
        return len(self.values)

    def clone(self):
        return Vec(*self.values, dtype=self.dtype)

    def __add__(self, other):
        return Vec(*(a + b for a, b in zip(self.values, other.values)))

    def __truediv__(self, k):
        return Vec(*(a / k for a in self.values))

    def __eq__(self, other):
        return isinstance(other, Vec) and self.values == other.values

    def __repr__(self):
        return f"Vec{self.values}"


class Slot:
    """A future stand-in."""

    def __init__(self):
        self.result = None

    def set_result(self, value):
        self.result = value


class Bucket:
    def __init__(self, tensor, index=0):
        self._tensor, self._index = tensor, index

    def index(self):
        return self._index

    def buffer(self):
        return self._tensor


PLAIN = CompressionConfig(bit=8, error_feedback=False)
WITH_FEEDBACK = CompressionConfig(bit=8, error_feedback=True, error_feedback_policy="always")


def two_ranks(n=2, names=("rank0", "rank1")):
    return GatheredPayloads(payloads=[CompressedPayload(buffer=name, shape=(n,), dtype="fp16") for name in names],
                            world_size=len(names))


class Log(list):
    def note(self, *item):
        self.append(item if len(item) > 1 else item[0])


# --------------------------------------------------------------------------- #
# all_reduce strategy
# --------------------------------------------------------------------------- #
def test_all_reduce_hook_resolves_a_future_and_hands_the_codec_output_through_unchanged():
    log = Log()

    def quantize(tensor, config):
        log.note("quantize", tensor, config.bit)
        return {"buffer": tensor, "shape": tensor.shape, "dtype": "fp16"}

    def dequantize(payload, shape, config, dtype):
        log.note("dequantize", payload, shape, dtype)
        return payload["buffer"]

    hook = create_ddp_comm_hook(PLAIN, dtype="fp16", quantize=quantize, dequantize=dequantize,
                                all_reduce=lambda payload, op: payload, future_factory=Slot)
    future = hook(state=None, bucket=Bucket(Vec(1, 2)))
    assert isinstance(future, Slot) and future.result == Vec(1, 2)
    assert log == [("quantize", Vec(1, 2), 8),
                   ("dequantize", {"buffer": Vec(1, 2), "shape": (2,), "dtype": "fp16"}, (2,), "fp16")]


def test_all_reduce_transport_sees_a_payload_and_the_sum_op():
    seen = []

    def all_reduce(payload, op):
        seen.append((payload.buffer, op))
        return payload.with_buffer({"buffer": Vec(3), "shape": payload.shape, "dtype": payload.dtype})

    hook = create_ddp_comm_hook(PLAIN, dtype="fp16",
                                quantize=lambda t, c: {"buffer": t, "shape": t.shape, "dtype": "fp16"},
                                dequantize=lambda p, shape, c, dtype: p["buffer"], all_reduce=all_reduce,
                                future_factory=Slot)
    assert hook(None, Bucket(Vec(1))).result == Vec(3)
    assert seen == [({"buffer": Vec(1), "shape": (1,), "dtype": "fp16"}, "sum")]


def test_bucket_dtype_is_inferred_from_the_tensor_when_not_given():
    seen = []
    hook = create_ddp_comm_hook(PLAIN, quantize=lambda t, c: t,
                                dequantize=lambda p, shape, c, dtype: seen.append(dtype) or p,
                                all_reduce=lambda p, op: p, future_factory=Slot)
    hook(None, Bucket(Vec(1, dtype="torch.float32")))
    hook(None, Bucket(Vec(1, dtype="torch.bfloat16")))
    assert seen == ["fp32", "bf16"]
    with pytest.raises(ValueError, match="cannot infer"):
        hook(None, Bucket(Vec(1, dtype="torch.int32")))


def test_annotations_come_from_the_provider():
    wanted = {"state": object, "bucket": "GradBucket", "return": "FutureTensor"}
    hook = create_ddp_comm_hook(PLAIN, dtype="fp16", quantize=lambda t, c: t, dequantize=lambda p, s, c, d: p,
                                all_reduce=lambda p, op: p, future_factory=Slot, annotation_provider=lambda: dict(wanted))
    assert hook.__annotations__ == wanted


# --------------------------------------------------------------------------- #
# strategy resolution and injected whole-collective transports
# --------------------------------------------------------------------------- #
def test_auto_strategy_resolves_to_all_gather_and_says_so():
    hook = create_ddp_comm_hook(PLAIN, dtype="fp16", strategy="auto",
                                quantize=lambda t, c: CompressedPayload(buffer=t, shape=t.shape, dtype="fp16"),
                                dequantize=lambda p, s, c, d: p.buffer,
                                all_gather=lambda p: GatheredPayloads(payloads=[p, p], world_size=2), future_factory=Slot)
    plan = hook._ccdl_strategy_plan
    assert (plan.requested_strategy, plan.strategy, plan.fallback_strategy) == ("auto", "all_gather", "all_gather")
    assert hook._ccdl_effective_strategy == "all_gather"


@pytest.mark.parametrize("strategy,keyword,answer", [
    ("hierarchical", "hierarchical_all_reduce", Vec(7, 9)),
    ("reduce_scatter", "reduce_scatter_all_gather", Vec(11, 13)),
    ("topology", "topology_all_reduce", Vec(17, 19)),
])
def test_whole_collective_transports_get_the_bucket_and_the_keyword_contract(strategy, keyword, answer):
    seen = []

    def transport(tensor, *, config, op, async_op, dtype, extension_status):
        seen.append((tensor, config.bit, op, async_op, dtype, extension_status))
        return answer

    hook = create_ddp_comm_hook(PLAIN, dtype="fp16", strategy=strategy, future_factory=Slot, **{keyword: transport})
    assert hook(None, Bucket(Vec(1, 2))).result == answer
    assert hook._ccdl_effective_strategy == strategy and hook._ccdl_strategy_plan.requires_fallback is False
    assert seen == [(Vec(1, 2), 8, "mean", False, "fp16", None)]


@pytest.mark.parametrize("strategy", ("hierarchical", "reduce_scatter"))
def test_an_explicit_strategy_without_its_transport_is_refused_when_the_hook_is_built(strategy):
    with pytest.raises(UnsupportedCollective, match=strategy):
        create_ddp_comm_hook(PLAIN, dtype="fp16", strategy=strategy, future_factory=Slot)
    with pytest.raises(UnsupportedCollective):
        create_ddp_comm_hook(PLAIN, dtype="fp16", strategy="ring-of-rings", future_factory=Slot)


# --------------------------------------------------------------------------- #
# all_gather strategy, synchronous
# --------------------------------------------------------------------------- #
def test_all_gather_mean_with_a_custom_decoder_decodes_every_rank_and_averages():
    log = Log()

    def all_gather(payload):
        log.note("all_gather", payload.buffer)
        return GatheredPayloads(payloads=[CompressedPayload(buffer=Vec(2), shape=(1,), dtype="fp16"),
                                          CompressedPayload(buffer=Vec(4), shape=(1,), dtype="fp16")], world_size=2)

    def dequantize(payload, shape, config, dtype):
        log.note("dequantize", payload.buffer, shape, dtype)
        return payload.buffer

    hook = create_ddp_comm_hook(PLAIN, dtype="fp16", strategy="all_gather", reduce="mean",
                                quantize=lambda t, c: log.note("quantize", t) or t, dequantize=dequantize,
                                all_gather=all_gather, future_factory=Slot)
    assert hook(None, Bucket(Vec(1))).result == Vec(3)
    assert log == [("quantize", Vec(1)), ("all_gather", Vec(1)), ("dequantize", Vec(2), (1,), "fp16"),
                   ("dequantize", Vec(4), (1,), "fp16")]


def test_a_bare_codec_buffer_is_wrapped_before_the_gather_and_payload_metadata_survives_it():
    log = Log()

    def quantize(tensor, config):
        return CompressedPayload(buffer=tensor, shape=tensor.shape, dtype="fp16", metadata={"original_numel": tensor.numel()})

    def gather(payload):
        log.note("all_gather", payload.buffer)
        return GatheredPayloads(payloads=[payload, payload], world_size=2)

    def dequantize(payload, shape, config, dtype):
        log.note("dequantize", payload.buffer, payload.metadata.get("original_numel"), payload.shape, payload.dtype)
        return payload.buffer

    hook = create_ddp_comm_hook(PLAIN, dtype="fp16", strategy="all_gather", quantize=quantize, dequantize=dequantize,
                                all_gather=gather, fuse_payload=True, fuse_payload_min_numel=4_000_000, future_factory=Slot)
    assert hook(None, Bucket(Vec(1, 2))).result == Vec(1, 2)
    assert log == [("all_gather", Vec(1, 2)), ("dequantize", Vec(1, 2), 2, (2,), "fp16"),
                   ("dequantize", Vec(1, 2), 2, (2,), "fp16")]
    log.clear()
    bare = create_ddp_comm_hook(PLAIN, dtype="fp16", strategy="all_gather", quantize=lambda t, c: t,
                                dequantize=dequantize, all_gather=gather, future_factory=Slot)
    assert bare(None, Bucket(Vec(1, 2))).result == Vec(1, 2)
    assert log == [("all_gather", Vec(1, 2)), ("dequantize", Vec(1, 2), None, (2,), "fp16"),
                   ("dequantize", Vec(1, 2), None, (2,), "fp16")]


def test_small_buckets_skip_the_codec_and_go_to_the_uncompressed_all_reduce():
    seen = []

    def refuse(*args, **kwargs):
        raise AssertionError("a small bucket must not reach the codec")

    hook = create_ddp_comm_hook(CompressionConfig(bit=8, error_feedback=True), dtype="fp16", strategy="all_gather",
                                reduce="mean", min_compress_numel=4, quantize=refuse, dequantize=refuse,
                                all_gather=refuse, bypass_all_reduce=lambda t, op: seen.append((t, op)) or Vec(3, 5),
                                future_factory=Slot)
    assert hook(None, Bucket(Vec(1, 2))).result == Vec(3, 5)
    assert seen == [(Vec(1, 2), "mean")]


def test_without_a_custom_decoder_the_fused_decode_reduce_of_the_facade_runs_once(monkeypatch):
    log = Log()
    monkeypatch.setattr(hook_module, "dequantize_reduce_tensors",
                        lambda buffers, shape, config, **kw: log.note("reduce", buffers, shape, kw["dtype"], kw["reduce"]) or Vec(2, 4))
    hook = create_ddp_comm_hook(PLAIN, dtype="fp16", strategy="all_gather", reduce="mean",
                                quantize=lambda t, c: CompressedPayload(buffer="local", shape=t.shape, dtype="fp16"),
                                all_gather=lambda p: two_ranks(), future_factory=Slot)
    assert hook(None, Bucket(Vec(1, 2))).result == Vec(2, 4)
    assert log == [("reduce", ["rank0", "rank1"], (2,), "fp16", "mean")]


class RecordingFeedback:
    """compensate / update only - the smallest feedback object the hook accepts."""

    def __init__(self, log, prepared):
        self.log, self.prepared = log, prepared

    def compensate(self, key, tensor):
        self.log.note("compensate", key, tensor)
        return self.prepared

    def update(self, key, *, original, transmitted):
        self.log.note("update", key, original, transmitted)


@pytest.mark.parametrize("numel,applies", [(2, False), (4, True)])
def test_large_bucket_only_policy_gates_compensate_and_update(monkeypatch, numel, applies):
    log = Log()
    monkeypatch.setattr(hook_module, "dequantize_reduce_tensors", lambda *a, **k: Vec(*range(2, 2 + numel)))
    config = CompressionConfig(bit=8, error_feedback=True, error_feedback_policy="large_bucket_only",
                               error_feedback_min_numel=4)
    prepared = Vec(*range(10, 10 + numel))
    hook = create_ddp_comm_hook(config, dtype="fp16", strategy="all_gather", reduce="mean",
                                quantize=lambda t, c: log.note("quantize", t) or CompressedPayload(buffer="local", shape=t.shape, dtype="fp16"),
                                all_gather=lambda p: two_ranks(numel), error_feedback=RecordingFeedback(log, prepared),
                                future_factory=Slot)
    bucket = Vec(*range(1, 1 + numel))
    hook(None, Bucket(bucket))
    if applies:
        assert ("compensate", 0, bucket) in log and ("quantize", prepared) in log
        assert ("update", 0, prepared, Vec(*range(2, 2 + numel))) in log
    else:
        assert ("quantize", bucket) in log
        assert not [item for item in log if item[0] in ("compensate", "update")]


# --------------------------------------------------------------------------- #
# all_gather strategy, asynchronous gather
# --------------------------------------------------------------------------- #
class GatherWork:
    """What an asynchronous gather returns: a future to chain on and a blocking ``wait``."""

    def __init__(self, log, numel=2):
        self.log, self.numel = log, numel

    def get_future(self):
        self.log.note("get_future")
        log = self.log

        class Chain:
            def then(self, callback):
                log.note("then")
                return callback(self)

        return Chain()

    def wait(self):
        self.log.note("wait")
        return two_ranks(self.numel)


class Completions:
    def __init__(self, log):
        self.log = log

    def record_for(self, tensor):
        self.log.note("record", tensor)
        log = self.log

        class Done:
            def wait(self):
                log.note("completion_wait")

            def synchronize(self):
                log.note("completion_synchronize")

        return Done()


def async_hook(log, config, *, feedback=None, reduce_result=Vec(2, 4, 6, 8), numel=4, **extra):
    def quantize(tensor, cfg):
        log.note("quantize", tensor)
        return CompressedPayload(buffer="local", shape=tensor.shape, dtype="fp16")

    def async_all_gather(buffer):
        log.note("async_all_gather", buffer)
        return GatherWork(log, numel)

    return create_ddp_comm_hook(config, dtype="fp16", strategy="all_gather", reduce="mean", quantize=quantize,
                                async_gather=True, async_all_gather=async_all_gather, error_feedback=feedback,
                                future_factory=Slot, **extra)


def test_async_gather_completes_the_bucket_from_the_gather_future(monkeypatch):
    log = Log()
    monkeypatch.setattr(hook_module, "dequantize_reduce_tensors",
                        lambda buffers, shape, config, **kw: log.note("reduce", buffers, kw["reduce"]) or Vec(2, 4))
    hook = async_hook(log, PLAIN, numel=2)
    assert hook(None, Bucket(Vec(1, 2))).result == Vec(2, 4)
    assert log == [("quantize", Vec(1, 2)), ("async_all_gather", "local"), "get_future", "then", "wait",
                   ("reduce", ["rank0", "rank1"], "mean")]


def test_async_gather_needs_its_transport():
    with pytest.raises(UnsupportedCollective, match="async"):
        create_ddp_comm_hook(PLAIN, dtype="fp16", strategy="all_gather", async_gather=True, future_factory=Slot)


def test_feedback_buckets_stay_synchronous_unless_async_feedback_is_requested(monkeypatch):
    log = Log()
    monkeypatch.setattr(hook_module, "dequantize_reduce_tensors",
                        lambda buffers, shape, config, **kw: log.note("reduce", buffers, kw["reduce"]) or Vec(2, 4, 6, 8))

    def sync_gather(payload):
        log.note("all_gather", payload.buffer)
        return two_ranks(4)

    def refuse(buffer):
        raise AssertionError("a bucket with error feedback must use the synchronous gather here")

    prepared = Vec(10, 20, 30, 40)
    hook = create_ddp_comm_hook(WITH_FEEDBACK, dtype="fp16", strategy="all_gather", reduce="mean",
                                quantize=lambda t, c: log.note("quantize", t) or CompressedPayload(buffer="local", shape=t.shape, dtype="fp16"),
                                all_gather=sync_gather, async_gather=True, async_all_gather=refuse,
                                error_feedback=RecordingFeedback(log, prepared), future_factory=Slot)
    assert hook(None, Bucket(Vec(1, 2, 3, 4))).result == Vec(2, 4, 6, 8)
    assert log == [("compensate", 0, Vec(1, 2, 3, 4)), ("quantize", prepared), ("all_gather", "local"),
                   ("reduce", ["rank0", "rank1"], "mean"), ("update", 0, prepared, Vec(2, 4, 6, 8))]


def test_async_feedback_pipeline_orders_decode_update_and_completion(monkeypatch):
    log = Log()
    monkeypatch.setattr(hook_module, "dequantize_reduce_tensors",
                        lambda buffers, shape, config, **kw: log.note("reduce", buffers, kw["reduce"]) or Vec(2, 4, 6, 8))
    prepared = Vec(10, 20, 30, 40)
    hook = async_hook(log, WITH_FEEDBACK, feedback=RecordingFeedback(log, prepared), async_error_feedback=True,
                      completion_manager=Completions(log))
    assert hook(None, Bucket(Vec(1, 2, 3, 4))).result == Vec(2, 4, 6, 8)
    assert log == [("compensate", 0, Vec(1, 2, 3, 4)), ("quantize", prepared), ("async_all_gather", "local"),
                   "get_future", "then", "wait", ("reduce", ["rank0", "rank1"], "mean"),
                   ("update", 0, prepared, Vec(2, 4, 6, 8)), ("record", Vec(2, 4, 6, 8)), "completion_wait",
                   "completion_synchronize"]


def test_host_side_completion_wait_can_be_switched_off(monkeypatch):
    log = Log()
    monkeypatch.setattr(hook_module, "dequantize_reduce_tensors", lambda *a, **k: Vec(2, 4, 6, 8))
    hook = async_hook(log, WITH_FEEDBACK, feedback=RecordingFeedback(log, Vec(10, 20, 30, 40)),
                      async_error_feedback=True, completion_manager=Completions(log),
                      synchronize_async_feedback_completion=False)
    hook(None, Bucket(Vec(1, 2, 3, 4)))
    assert "completion_wait" in log and "completion_synchronize" not in log


class StoredFeedback(RecordingFeedback):
    """Feedback that also exposes the stored residual, which unlocks the native update paths."""

    def __init__(self, log, prepared, residual):
        super().__init__(log, prepared)
        self.residual = residual

    def update(self, key, *, original, transmitted):
        raise AssertionError("a native update must replace the Python residual update")

    def get(self, key):
        self.log.note("get", key)
        return self.residual


def test_native_residual_update_replaces_the_python_one(monkeypatch):
    log = Log()
    monkeypatch.setattr(hook_module, "dequantize_reduce_tensors", lambda *a, **k: Vec(2, 4, 6, 8))
    residual, prepared = Vec(.5, .5, .5, .5), Vec(1.5, 2.5, 3.5, 4.5)
    hook = async_hook(log, WITH_FEEDBACK, feedback=StoredFeedback(log, prepared, residual), async_error_feedback=True,
                      completion_manager=Completions(log),
                      native_error_feedback_update=lambda p, r, existing: log.note("native_update", p, r, existing))
    assert hook(None, Bucket(Vec(1, 2, 3, 4))).result == Vec(2, 4, 6, 8)
    assert ("native_update", prepared, Vec(2, 4, 6, 8), residual) in log and ("get", 0) in log


def test_combined_native_reduce_and_update_replaces_both_steps(monkeypatch):
    log = Log()

    def refuse(*a, **k):
        raise AssertionError("the combined native call must replace the separate decode-reduce")

    monkeypatch.setattr(hook_module, "dequantize_reduce_tensors", refuse)
    residual, prepared = Vec(.5, .5, .5, .5), Vec(1.5, 2.5, 3.5, 4.5)

    def combined(buffers, prepared_, existing, shape, config, **kw):
        log.note("combined", buffers, prepared_, existing, shape, kw["dtype"], kw["reduce"])
        return Vec(2, 4, 6, 8)

    hook = async_hook(log, WITH_FEEDBACK, feedback=StoredFeedback(log, prepared, residual), async_error_feedback=True,
                      completion_manager=Completions(log), native_dequantize_reduce_update_feedback=combined)
    assert hook(None, Bucket(Vec(1, 2, 3, 4))).result == Vec(2, 4, 6, 8)
    assert ("combined", ["rank0", "rank1"], prepared, residual, (4,), "fp16", "mean") in log


def workspace_hook(log, monkeypatch, *, buckets=1, **extra):
    def refuse(*a, **k):
        raise AssertionError("the in-place fused call must replace the separate decode-reduce")

    monkeypatch.setattr(hook_module, "dequantize_reduce_tensors", refuse)
    residual, prepared = Vec(.5, .5, .5, .5), Vec(1.5, 2.5, 3.5, 4.5)
    made = []

    def allocate(tensor, shape, config):
        workspace = Vec(0, 0, 0, 0)
        made.append(workspace)
        log.note("allocate", tensor, shape, config.group_size)
        return workspace

    def fused(buffers, prepared_, restored, existing, config, **kw):
        log.note("fused", buffers, prepared_, restored is made[-1] or restored in made, existing, kw["reduce"])
        return True

    hook = async_hook(log, WITH_FEEDBACK, feedback=StoredFeedback(log, prepared, residual), async_error_feedback=True,
                      completion_manager=Completions(log), native_inplace_dequantize_reduce_update_feedback=fused,
                      allocate_dequantized_workspace=allocate, **extra)
    return hook, made, prepared, residual


def test_in_place_fused_feedback_writes_into_a_cached_workspace(monkeypatch):
    log = Log()
    hook, made, prepared, residual = workspace_hook(log, monkeypatch)
    first = hook(None, Bucket(Vec(1, 2, 3, 4)))
    second = hook(None, Bucket(Vec(1, 2, 3, 4)))
    assert first.result is made[0] and second.result is made[0]          # the workspace itself, reused
    assert log.count(("allocate", prepared, (4,), 64)) == 1
    assert log.count(("fused", ["rank0", "rank1"], prepared, True, residual, "mean")) == 2


def test_workspace_cache_holds_one_entry_unless_told_otherwise(monkeypatch):
    log = Log()
    hook, made, _, _ = workspace_hook(log, monkeypatch)
    for index in (0, 1, 0):
        hook(None, Bucket(Vec(1, 2, 3, 4), index=index))
    assert len(made) == 3                                                  # bucket 0 was evicted by bucket 1
    log = Log()
    roomy, made, _, _ = workspace_hook(log, monkeypatch, workspace_cache_max_entries=2)
    for index in (0, 1, 0):
        roomy(None, Bucket(Vec(1, 2, 3, 4), index=index))
    assert len(made) == 2


# --------------------------------------------------------------------------- #
# the bucket processor on its own
# --------------------------------------------------------------------------- #
def test_processor_hands_the_bucket_view_to_the_codec_and_applies_feedback_first():
    log = Log()
    processor = DDPBucketProcessor(
        config=PLAIN, quantize=lambda t, c: log.note("quantize", t, c.bit) or {"buffer": t},
        dequantize=lambda p, shape, c, dtype: log.note("dequantize", p, shape, dtype) or p["buffer"])
    assert processor.process(Bucket(Vec(1, 2)), dtype="bf16") == Vec(1, 2)
    assert log == [("quantize", Vec(1, 2), 8), ("dequantize", {"buffer": Vec(1, 2)}, (2,), "bf16")]

    log.clear()
    with_feedback = DDPBucketProcessor(config=WITH_FEEDBACK, quantize=lambda t, c: log.note("quantize", t) or t,
                                       dequantize=lambda p, shape, c, dtype: Vec(9, 9),
                                       error_feedback=RecordingFeedback(log, Vec(10, 20)))
    assert with_feedback.process(Bucket(Vec(1, 2), index=5), dtype="fp16") == Vec(9, 9)
    assert log == [("compensate", 5, Vec(1, 2)), ("quantize", Vec(10, 20)), ("update", 5, Vec(10, 20), Vec(9, 9))]


def test_processor_uses_an_injected_all_reduce_and_builds_from_a_native_codec():
    seen = []

    def all_reduce(payload, op):
        seen.append((payload.buffer, payload.shape, payload.dtype, op))
        return payload.with_buffer("reduced")

    processor = DDPBucketProcessor(config=PLAIN, quantize=lambda t, c: "local", dequantize=lambda p, shape, c, d: p,
                                   all_reduce=all_reduce)
    assert processor.process(Bucket(Vec(1, 2)), dtype="fp16") == "reduced"
    assert seen == [("local", (2,), "fp16", "sum")]

    class Status:
        available, module, reason = True, object(), None

    built = DDPBucketProcessor.from_cuda_codec(PLAIN, extension_status=Status())
    assert built.config is PLAIN and callable(built.quantize) and callable(built.dequantize)
