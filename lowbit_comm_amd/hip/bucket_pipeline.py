"""A stream of gradient buckets through the compressed reduce-scatter (+ all-gather) plan, software-pipelined.

The reference's transport is a pipeline: while bucket k is quantized, the exchange of bucket k-1 is in flight, and what
completes that exchange is the reduce of its shard (``ccdl_comm/communication/reduce_scatter_transport.py:262-347``,
``ccdl_comm/communication/async_shard_pipeline.py:11-129``); the topology family continues with requantize, all-gather
and the decode of every shard (``ccdl_comm/communication/topology_transport.py:866-894``).  Consecutive DDP buckets are
independent of each other, so at any moment three compute stages of three different buckets are ready together:

    bucket k     quantize + pack of its W chunks (optionally with error feedback)    then its all-to-all
    bucket k-1   reduce (+ requantize) of the W payloads that arrived for its shard   then its all-gather
    bucket k-2   decode of its W gathered shard payloads                              then its future completes

:class:`BucketPipeline` issues them as ONE launch per bucket (``lbc_bucket_pipeline_step`` for the full plan,
``lbc_quant_pack_chunks_and_dequant_reduce`` for the reduce-scatter leg alone): on this part the shard-sized stages
are mostly launch ramp on their own, and behind a quantize that fills the chip that ramp is hidden (25 MiB bf16 buckets
with error feedback, W = 8: 31 us per bucket in one grid against 37 us as three launches).  When a combination has no
shared grid (unaligned tensors, a group size other than 64, more than eight ranks) the same stages go out as separate launches,
in the same order, with the same results.

Ordering.  Everything is enqueued on the caller's current stream (or on the pipeline's lanes, see ``lanes``), so a
stage is ordered after the exchange it depends on by the stream itself when the exchange callables enqueue on that
stream; an exchange that returns a work object (``wait()``) is waited for - a stream wait for ``torch.distributed``
work, not a host wait - right before the launch that reads what it delivers.  Each bucket in flight owns one of three
(two, for the reduce-scatter leg alone) plans of its shape, so nothing a launch writes is read by a stage of another
bucket in the same launch.

Completion.  A bucket's future is completed when its last launch has been *enqueued* - with the next bucket but one,
or by :meth:`flush`.  The DDP hook flushes when it has been handed the iteration's last bucket
(``GradBucket.is_last()``); the futures made here flush by themselves when somebody waits for them.
"""
from __future__ import annotations

import threading
from collections import OrderedDict
from collections.abc import Callable
from typing import Any

import torch

from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.hip import ops
from lowbit_comm_amd.hip.reduce_scatter import AllGatherPlan, ReduceScatterPlan, ResidualStore


class _Bucket:
    """One bucket in flight: its plan (send / received / gathered rows), tensors, future and pending exchanges."""

    __slots__ = ("plan", "tensor", "out", "op", "future", "exchange", "gather", "result", "lane", "lasting_out", "spans")

    def __init__(self, plan: ReduceScatterPlan, tensor: torch.Tensor, out: torch.Tensor | None, op: str, future: Any,
                 lane: int, lasting_out: bool, spans: tuple) -> None:
        self.plan = plan
        self.tensor = tensor
        self.out = out
        self.op = op
        self.future = future
        self.lasting_out = lasting_out        # the output is memory that will come back (the bucket itself, the caller's)
        self.exchange: Any | None = None      # work object of the all-to-all, if it returned one
        self.gather: Any | None = None        # work object of the all-gather, if it returned one
        self.result: Any | None = None
        self.lane = lane
        self.spans = spans                    # byte ranges this bucket reads and writes while it is in flight


def _span(tensor: torch.Tensor) -> tuple[int, int]:
    start = tensor.data_ptr()
    return start, start + tensor.numel() * tensor.element_size()


def _wait_for(work: Any) -> None:
    wait = getattr(work, "wait", None)
    if callable(wait):
        wait()


class _Lane:
    """The buckets of one stream: at most one awaiting its reduce and one awaiting its decode."""

    __slots__ = ("stream", "handle", "reduce_next", "decode_next", "ready")

    def __init__(self, stream: Any | None) -> None:
        self.stream = stream
        self.handle = None if stream is None else stream.cuda_stream
        self.reduce_next: _Bucket | None = None
        self.decode_next: _Bucket | None = None
        self.ready = None if stream is None else torch.cuda.Event()    # "the caller's stream has got this far", reused


class BucketPipeline:
    """``submit(tensor, config=..., op=...)`` per bucket, in arrival order; ``flush()`` after the last one.

    ``all_to_all(received_rows, send_rows)`` and ``all_gather(gathered_rows, my_payload)`` are the two exchanges of
    :func:`~lowbit_comm_amd.hip.reduce_scatter.compressed_all_reduce_via_reduce_scatter`; each may return a work object.
    Without ``all_gather`` the pipeline stops after the reduce-scatter leg: a bucket's future then resolves to its
    :class:`~lowbit_comm_amd.shard.ReducedShard` (in ``out=`` of :meth:`submit`, else in a fresh tensor).  With it, the
    future resolves to the reduced bucket - decoded in place into ``tensor`` when ``inplace`` and the tensor is
    contiguous, else into a fresh tensor.

    ``whole_gather(received_rows, my_payload)`` instead of ``all_to_all`` selects the all-gather form of the all-reduce
    (the comm hook's ``all_gather`` strategy, ``ccdl_comm/communication/ddp_hook.py:190-330``): a bucket is quantized
    into one payload, the ``W`` payloads are all-gathered and one fused launch reduces them into the bucket.  The
    quantize of bucket k then shares its launch with the reduce of bucket k-1, and a future resolves to the reduced
    bucket (in place under the same condition as above).

    ``error_feedback``: every bucket (keyed by storage address, element count and dtype) keeps an fp32 residual that
    its quantize adds before encoding and refreshes, in the same launch, with what the encoding dropped; beyond
    ``max_residuals`` buckets the least recently used residual is dropped.

    ``lanes`` > 1 deals the buckets to that many streams of default priority in turn, each with its own buckets in
    flight: the ramp-up of one bucket's launch overlaps the drain of the one before.  A lane waits for the caller's
    stream before it touches a bucket, and :meth:`flush` makes the caller's stream wait for every lane; a future
    completed before the flush says that the work has been enqueued on a lane, not that the caller's stream is ordered
    after it.

    Calls from several threads are serialised by a lock; the buckets of one iteration still have to arrive in one
    order."""

    def __init__(self, *, world_size: int, rank: int, all_to_all: Callable[[torch.Tensor, torch.Tensor], Any] | None = None,
                 all_gather: Callable[[torch.Tensor, torch.Tensor], Any] | None = None, error_feedback: bool = False,
                 inplace: bool = True, lanes: int = 1, max_plans: int = 64, max_steps: int = 4096,
                 future_factory: Callable[[], Any] | None = None, plan_factory: Callable[..., Any] | None = None,
                 merge_stages: Callable[..., Any] | None = None, max_residuals: int = 4096,
                 whole_gather: Callable[[torch.Tensor, torch.Tensor], Any] | None = None) -> None:
        if not 0 <= rank < world_size:
            raise ValueError(f"rank must be in [0, {world_size})")
        if lanes < 1:
            raise ValueError("lanes must be at least 1")
        if (all_to_all is None) == (whole_gather is None):
            raise ValueError("give either all_to_all (reduce-scatter form) or whole_gather (all-gather form)")
        if whole_gather is not None and all_gather is not None:
            raise ValueError("the all-gather form has one exchange: whole_gather")
        self.world_size = world_size
        self.rank = rank
        self.all_to_all = all_to_all
        self.all_gather = all_gather
        self.whole_gather = whole_gather
        self.error_feedback = bool(error_feedback)
        self.inplace = bool(inplace)
        self.depth = 3 if all_gather is not None else 2
        self.max_plans = max_plans
        self.max_steps = max_steps
        self.residuals = ResidualStore(max_residuals)
        self.stats = {"buckets": 0, "merged_launches": 0, "separate_launches": 0, "flushes": 0}
        self._future_factory = future_factory
        # replaceable: the scheduling is testable without a GPU
        self._plan_factory = plan_factory or (AllGatherPlan if whole_gather is not None else ReduceScatterPlan)
        self._merge_stages = merge_stages or self._bind_merged
        self._dirty = False                                        # something was submitted since the last flush
        self._lock = threading.RLock()
        self._plans: OrderedDict[Any, list[ReduceScatterPlan]] = OrderedDict()   # shape key -> `depth` plans per lane
        self._turn: dict[Any, int] = {}                                          # shape key -> buckets seen since flush
        self._steps: OrderedDict[Any, tuple] = OrderedDict()                     # merged launches, by their parts
        self._lane_count = lanes
        self._lanes: list[_Lane] | None = None
        self._next_lane = 0

    # ---- bookkeeping ------------------------------------------------------------------------------
    @property
    def pending(self) -> int:
        """Buckets whose future has not been completed yet."""
        if self._lanes is None:
            return 0
        return sum((lane.reduce_next is not None) + (lane.decode_next is not None) for lane in self._lanes)

    def reset(self) -> None:
        """Drop the error-feedback residuals (after a flush)."""
        self.flush()
        self.residuals.clear()

    def make_future(self) -> Any:
        """A future of the configured kind; the default kind flushes the pipeline when it is waited for unfinished."""
        if self._future_factory is not None:
            return self._future_factory()
        return _FlushingFuture(self.flush)

    def _lanes_for(self, device: torch.device) -> list[_Lane]:
        if self._lanes is None:
            if self._lane_count == 1:
                self._lanes = [_Lane(None)]
            else:
                self._lanes = [_Lane(torch.cuda.Stream(device=device)) for _ in range(self._lane_count)]   # default priority
        return self._lanes

    def _residual_for(self, tensor: torch.Tensor) -> torch.Tensor | None:
        return self.residuals.for_tensor(tensor) if self.error_feedback else None

    def _touches_a_bucket_in_flight(self, mine: tuple) -> bool:
        for lane in self._lanes or ():
            for bucket in (lane.reduce_next, lane.decode_next):
                if bucket is None:
                    continue
                for low, high in bucket.spans:
                    for a, b in mine:
                        if low < b and a < high:
                            return True
        return False

    def _plan_for(self, tensor: torch.Tensor, config: CompressionConfig, lane: int) -> ReduceScatterPlan:
        key = (tensor.numel(), tensor.dtype, tensor.device, config.bit, config.group_size, config.topk,
               config.quant_type, config.stochastic)
        ring = self._plans.get(key)
        if ring is None:
            ring = self._plans[key] = [
                self._plan_factory(tensor.numel(), tensor.dtype, world_size=self.world_size, rank=self.rank, config=config,
                                   device=tensor.device, shape=tuple(tensor.shape))
                for _ in range(self.depth * self._lane_count)]
            while len(self._plans) > self.max_plans:
                old_key, _ = self._plans.popitem(last=False)
                for turn_key in [k for k in self._turn if k[0] == old_key]:
                    del self._turn[turn_key]
        else:
            self._plans.move_to_end(key)
        # the turn counts this lane's buckets of this shape since the last flush, so a bucket meets the same plan
        # again in the next iteration and its bound launches are found again
        turn_key = (key, lane)
        turn = self._turn.get(turn_key, 0)
        self._turn[turn_key] = turn + 1
        return ring[lane * self.depth + turn % self.depth]

    # ---- one step ---------------------------------------------------------------------------------
    def _merged(self, quant: ops.BoundLaunch | None, reduce: ops.BoundLaunch | None, decode: ops.BoundLaunch | None):
        """The one-launch form of the given stages, remembered by their identity; ``None`` when there is none."""
        key = (id(quant), id(reduce), id(decode))
        entry = self._steps.get(key)
        if entry is not None and entry[0] is quant and entry[1] is reduce and entry[2] is decode:
            self._steps.move_to_end(key)
            return entry[3]
        step = self._merge_stages(quant, reduce, decode)
        self._steps[key] = (quant, reduce, decode, step)      # the parts are kept alive: their ids stay theirs
        while len(self._steps) > self.max_steps:
            self._steps.popitem(last=False)
        return step

    def _bind_merged(self, quant, reduce, decode):
        if self.all_gather is not None:
            return ops.bind_bucket_pipeline_step(quant, reduce, decode)
        return ops.bind_quant_chunks_and_reduce(quant, reduce)

    def _launch(self, lane: _Lane, quant, reduce, decode) -> None:
        parts = [part for part in (quant, reduce, decode) if part is not None]
        if not parts:
            return
        if len(parts) == 1:
            if not parts[0](lane.handle):
                raise ValueError("no HIP kernel for this stage")
            self.stats["separate_launches"] += 1
            return
        if self._merged(quant, reduce, decode)(lane.handle):
            self.stats["merged_launches"] += 1
            return
        for part in parts:                    # no shared grid for this combination: the same stages, one by one
            if not part(lane.handle):
                raise ValueError("no HIP kernel for this stage")
            self.stats["separate_launches"] += 1

    def _advance(self, lane: _Lane, arriving: _Bucket | None, residual: torch.Tensor | None) -> None:
        """One pipeline step on ``lane``: the stages that are ready, their exchanges, the completion of the oldest."""
        reducing, decoding = lane.reduce_next, lane.decode_next
        full = self.all_gather is not None
        quant = reduce = decode = None
        if arriving is not None:
            arriving.plan._order_after_previous_use()
            quant = arriving.plan.bound_quantize(arriving.tensor, residual=residual, new_residual=residual)
        if reducing is not None:
            _wait_for(reducing.exchange)
            reducing.exchange = None
            if full:
                reduce = reducing.plan.bound_reduce_requantize(op=reducing.op)
            else:
                reduce = reducing.plan.bound_reduce(op=reducing.op, out=reducing.out)
        if decoding is not None:
            _wait_for(decoding.gather)
            decoding.gather = None
            decode = decoding.plan.bound_decode(decoding.out, remember=decoding.lasting_out)
        self._launch(lane, quant, reduce, decode)
        if arriving is not None:
            if self.whole_gather is not None:
                arriving.exchange = self.whole_gather(arriving.plan.received, arriving.plan.my_payload)
            else:
                arriving.exchange = self.all_to_all(arriving.plan.received, arriving.plan.send)
        if reducing is not None:
            if full:
                reducing.gather = self.all_gather(reducing.plan.gathered, reducing.plan.my_row)
            elif self.whole_gather is not None:
                self._complete(reducing, reducing.out.reshape(reducing.tensor.shape))
            else:
                self._complete(reducing, reducing.plan.reduced_shard(reducing.out, op=reducing.op, caller_owned=True))
        if decoding is not None:
            self._complete(decoding, decoding.out.reshape(decoding.plan.shape))
        lane.decode_next = reducing if full else None
        lane.reduce_next = arriving

    @staticmethod
    def _complete(bucket: _Bucket, result: Any) -> None:
        bucket.result = result
        bucket.future.set_result(result)

    # ---- the caller's face ------------------------------------------------------------------------
    def submit(self, tensor: torch.Tensor, *, config: CompressionConfig, op: str = "mean",
               out: torch.Tensor | None = None) -> Any:
        """Hand over the next bucket; returns its future."""
        if op not in ("sum", "mean"):
            raise ValueError(f"unsupported reduce-scatter mode: {op}")
        with self._lock:
            future = self.make_future()
            self.stats["buckets"] += 1
            full = self.all_gather is not None
            whole = full or self.whole_gather is not None       # the result is the reduced bucket, not a shard
            if tensor.numel() == 0:           # nothing to exchange on any rank
                future.set_result(tensor if whole else
                                  self._plan_factory(0, tensor.dtype, world_size=self.world_size, rank=self.rank, config=config,
                                                     device=tensor.device, shape=tuple(tensor.shape))
                                  .reduced_shard(tensor.reshape(-1), op=op, fused=False, caller_owned=True))
                return future
            if self.world_size > ops.MAX_PAYLOADS:
                raise ValueError(f"the bucket pipeline reduces at most {ops.MAX_PAYLOADS} ranks in one launch; use the "
                                 "unpipelined plan beyond")
            lanes = self._lanes_for(tensor.device)
            index = self._next_lane
            self._next_lane = (index + 1) % len(lanes)
            lane = lanes[index]
            plan = self._plan_for(tensor, config, index)
            lasting_out = out is not None
            if whole:
                if out is None:
                    lasting_out = self.inplace and tensor.is_contiguous()
                    out = tensor.reshape(-1) if lasting_out else torch.empty(
                        tensor.numel(), dtype=plan.reduced_dtype, device=tensor.device)
                elif out.numel() != tensor.numel() or out.dtype != plan.reduced_dtype:
                    raise ValueError("out does not match the bucket")
            else:
                if out is None:
                    out = torch.empty(plan.chunks.shard_numel, dtype=plan.reduced_dtype, device=tensor.device)
                elif out.numel() != plan.chunks.shard_numel or out.dtype != plan.reduced_dtype:
                    raise ValueError("out does not match this rank's shard")
            spans = (_span(tensor),)
            if out.data_ptr() != spans[0][0] or out.numel() * out.element_size() != spans[0][1] - spans[0][0]:
                spans += (_span(out),)            # not the bucket itself: a second range
            if self._touches_a_bucket_in_flight(spans):
                # The same memory again before its earlier bucket has been decoded (not a DDP iteration, where every
                # bucket is handed over once): finish the earlier one first, so that this quantize reads its result
                # and no launch both reads and writes the tensor.
                self.flush()
                plan = self._plan_for(tensor, config, index)
            bucket = _Bucket(plan, tensor, out, op, future, index, lasting_out, spans)
            self._dirty = True
            residual = self._residual_for(tensor)
            if lane.stream is None:
                self._advance(lane, bucket, residual)
            else:
                current = torch.cuda.current_stream(tensor.device)
                lane.ready.record(current)                    # the bucket's gradients are ready on the caller's stream
                lane.stream.wait_event(lane.ready)
                torch.cuda.set_stream(lane.stream)            # the exchanges and the future see the lane as current
                try:
                    self._advance(lane, bucket, residual)
                finally:
                    torch.cuda.set_stream(current)
                # Every time, not once per address: a tensor that was freed and whose block was handed out again is a
                # new block to the caching allocator, which has to hear of the lane's use of it too.
                for held in (tensor, out) + (() if residual is None else (residual,)):
                    held.record_stream(lane.stream)
            return future

    def flush(self) -> None:
        """Issue what is left of the buckets in flight and complete their futures; with lanes, order the caller's
        stream after them.  Called by the DDP hook after the iteration's last bucket; cheap when nothing is pending."""
        with self._lock:
            lanes = self._lanes
            if lanes is None:
                return
            if not self._dirty:
                return
            self._turn.clear()
            self._next_lane = 0
            self.stats["flushes"] += 1
            for lane in lanes:
                if lane.stream is None:
                    while lane.reduce_next is not None or lane.decode_next is not None:
                        self._advance(lane, None, None)
                    continue
                current = torch.cuda.current_stream(lane.stream.device)
                torch.cuda.set_stream(lane.stream)
                try:
                    while lane.reduce_next is not None or lane.decode_next is not None:
                        self._advance(lane, None, None)
                finally:
                    torch.cuda.set_stream(current)
                current.wait_stream(lane.stream)
            self._dirty = False                   # only now: a flush that raised half-way is retried by the next one


class _FlushingFuture(torch.futures.Future):
    """A future of the pipeline: waiting for it first issues whatever the pipeline still holds back, so a caller that
    never flushes cannot wait for ever.  (DistributedDataParallel waits on the C++ side, where this override is not
    seen: the comm hook flushes after the last bucket instead.)"""

    def __init__(self, flush: Callable[[], None]) -> None:
        super().__init__()
        self._flush = flush

    def wait(self) -> Any:
        if not self.done():
            self._flush()
        return super().wait()

    def value(self) -> Any:
        if not self.done():
            self._flush()
        return super().value()


__all__ = ["BucketPipeline"]
