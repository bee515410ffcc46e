"""Compute steps of the compressed reduce-scatter (+ requantized all-gather) on one GPU.

The reference's transport (``ccdl_comm/communication/reduce_scatter_transport.py:186-377``) pads the
flattened bucket to ``W * shard_numel``, quantizes each destination chunk separately, exchanges the
payloads with an all-to-all, and reduces the ``W`` received payloads into this rank's shard; the
topology family then requantizes the shard, all-gathers the payloads and decodes every shard into
its slot (``ccdl_comm/communication/topology_transport.py:866-894``).  Here the exchange callables are
injected (or synthesised by a test / benchmark) and every compute step is one launch:

    quantize W chunks   -> lbc_quant_pack_chunks    (one launch for all W chunks)
    reduce W payloads   -> lbc_dequant_reduce        (fused, fixed rank order)
    requantize shard    -> lbc_quant_pack            (into row ``rank`` of the gather buffer)
    decode W shards     -> lbc_dequant_chunks        (one launch for all W shards)

Workspaces are allocated once per plan and reused, so a steady-state bucket allocates nothing.  A plan serves one
bucket at a time: uses on one stream are ordered by the stream, a use on another stream is ordered after the previous
one by an event, and a plan whose asynchronous exchange has not been waited for refuses the next bucket.
"""
from __future__ import annotations

import threading
from collections import OrderedDict
from collections.abc import Callable
from typing import Any

import torch

from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.hip import ops
from lowbit_comm_amd.hip.chunk_plan import ChunkPlan, compile_chunk_plan
from lowbit_comm_amd.hip.codec import ccdl_dtype, torch_dtype
from lowbit_comm_amd.shard import ReducedShard

_ROW_ALIGN = 256


class ReduceScatterPlan:
    """Pre-bound compute of one bucket shape at world size ``W`` for rank ``rank``."""

    def __init__(self, numel: int, dtype: torch.dtype, *, world_size: int, rank: int, config: CompressionConfig,
                 device: torch.device | str, reduced_dtype: torch.dtype | None = None,
                 shape: tuple[int, ...] | None = None) -> None:
        if config.bit != 8 or config.quant_type != "linear" or config.topk != 0 or config.stochastic:
            raise ValueError("the HIP reduce-scatter plan supports linear 8-bit quantization without top-k / stochastic")
        if not 0 <= rank < world_size:
            raise ValueError(f"rank must be in [0, {world_size})")
        self.config = config
        self.world_size = world_size
        self.rank = rank
        self.numel = int(numel)
        self.shape = tuple(shape) if shape is not None else (self.numel,)
        self.dtype = dtype
        self.reduced_dtype = reduced_dtype or dtype
        self.device = torch.device(device)
        self.chunks: ChunkPlan = compile_chunk_plan(original_numel=self.numel, world_size=world_size)
        shard = self.chunks.shard_numel
        g = config.group_size
        self.payload_bytes = ops.payload_nbytes(shard, g)
        self.row_stride = -(-self.payload_bytes // _ROW_ALIGN) * _ROW_ALIGN
        rows = (world_size, self.row_stride)
        self.send = torch.empty(rows, dtype=torch.uint8, device=self.device)       # my chunk for every rank
        self.received = torch.empty(rows, dtype=torch.uint8, device=self.device)   # every rank's chunk for me
        self.gathered = torch.empty(rows, dtype=torch.uint8, device=self.device)   # every rank's requantized shard
        self.shard = torch.empty(shard, dtype=self.reduced_dtype, device=self.device)
        self.my_row = self.gathered[rank, :self.payload_bytes]      # where this rank's requantized shard payload goes
        # Launches bound to the tensor addresses seen so far, least recently used dropped first.  Many buckets of one
        # shape share a plan (the layers of a transformer), so the cache is sized for them; its entries do not keep
        # the callers' tensors alive (the key holds everything a binding depends on, and every step is handed the
        # live tensors), so it pins no memory beyond the plan's own buffers.
        self._bound: OrderedDict[Any, ops.BoundLaunch] = OrderedDict()
        self._bound_lock = threading.Lock()   # DDP calls its hook from the autograd thread, a user may call from another
        self._last_stream: Any | None = None
        self._last_stream_handle: int | None = None
        self.exchange_in_flight: Any | None = None     # work object of an exchange that nobody has waited for yet

    # Every bucket of one shape shares the plan, and every bucket has its own addresses: a transformer's stream of
    # 25 MiB buckets has hundreds of them (613 for an 8 B-parameter model), each with up to three stages.  A cache
    # smaller than one pass over them would miss on every bucket.
    _BOUND_LAUNCHES = 4096

    def _remember(self, key: Any, make: Callable[[], ops.BoundLaunch]) -> ops.BoundLaunch:
        with self._bound_lock:
            bound = self._bound.get(key)
            if bound is not None:
                self._bound.move_to_end(key)
                return bound
        made = make().forget_tensors()           # binding validates tensors: outside the lock
        with self._bound_lock:
            bound = self._bound.setdefault(key, made)
            self._bound.move_to_end(key)
            while len(self._bound) > self._BOUND_LAUNCHES:
                self._bound.popitem(last=False)
        return bound

    def _order_after_previous_use(self) -> None:
        """Called by every step before it touches the plan's buffers.  On the stream of the previous step nothing is
        needed; on another stream an event recorded there now (it covers everything that stream was given so far,
        the previous step included) is waited for by the current stream."""
        if self.device.type != "cuda":
            return
        handle = ops.current_stream_handle(self.device)      # a raw handle: no stream object in the usual case
        if handle == self._last_stream_handle:
            return
        stream = torch.cuda.current_stream(self.device)
        if self._last_stream is not None:
            event = torch.cuda.Event()
            event.record(self._last_stream)                   # the stream object is kept, so its handle stays valid
            stream.wait_event(event)
        self._last_stream, self._last_stream_handle = stream, handle

    # ---- payload views ---------------------------------------------------------------------------
    def payload(self, rows: torch.Tensor, index: int) -> torch.Tensor:
        """Row ``index`` of a payload matrix, trimmed to the exact payload size (a view)."""
        return rows[index, :self.payload_bytes]

    def _pairs(self, rows: torch.Tensor):
        shard, g = self.chunks.shard_numel, self.config.group_size
        return [ops.split_payload(self.payload(rows, r), shard, g) for r in range(self.world_size)]

    # ---- compute steps ---------------------------------------------------------------------------
    def quantize_chunks(self, tensor: torch.Tensor, *, residual: torch.Tensor | None = None,
                        new_residual: torch.Tensor | None = None) -> torch.Tensor:
        """Quantize the ``W`` destination chunks of ``tensor`` (+ ``residual``) into ``self.send`` (one launch).

        With ``new_residual`` the same launch also stores what quantization dropped,
        ``(tensor + residual) - decode(payload)``; it may be the ``residual`` tensor itself."""
        bound = self.bound_quantize(tensor, residual=residual, new_residual=new_residual)
        self._order_after_previous_use()
        if self.numel and not bound():
            raise ValueError(f"no HIP quantize kernel for dtype {tensor.dtype} with this residual")
        return self.send

    def bound_quantize(self, tensor: torch.Tensor, *, residual: torch.Tensor | None = None,
                       new_residual: torch.Tensor | None = None) -> ops.BoundLaunch:
        """The launch of :meth:`quantize_chunks`, bound and remembered but not issued (a caller that merges the stages of
        several buckets into one launch takes it from here)."""
        flat = tensor.reshape(-1)
        if flat.numel() != self.numel or flat.dtype != self.dtype:
            raise ValueError("tensor does not match the planned bucket")
        if self.exchange_in_flight is not None:
            raise RuntimeError("this plan's send and receive buffers belong to an exchange that has not been waited for: "
                               "wait for the previous bucket's work first, or give every bucket in flight its own plan")
        key = ("q", flat.data_ptr(), None if residual is None else (residual.data_ptr(), residual.dtype, residual.numel()),
               None if new_residual is None else (new_residual.data_ptr(), new_residual.dtype, new_residual.numel()))
        return self._remember(key, lambda: ops.bind_quant_pack_chunks(
            flat, self.send, self.world_size, group_size=self.config.group_size,
            residual=None if residual is None else residual.reshape(-1),
            new_residual=None if new_residual is None else new_residual.reshape(-1)))

    def reduce_received(self, received: torch.Tensor | None = None, *, op: str = "sum",
                        out: torch.Tensor | None = None) -> ReducedShard:
        """Fused dequant-reduce of the ``W`` received payloads (rank order) into this rank's shard."""
        if op not in ("sum", "mean"):
            raise ValueError(f"unsupported reduce-scatter mode: {op}")
        rows = self.received if received is None else received
        target = self.shard if out is None else out
        shard = self.chunks.shard_numel
        fused = self.world_size <= ops.MAX_PAYLOADS
        self._order_after_previous_use()
        if shard:
            if fused:
                fused = bool(self.bound_reduce(rows, op=op, out=target)())
            if not fused:
                for r, (codes, scales) in enumerate(self._pairs(rows)):
                    ops.dequant_into(codes, scales, target, numel=shard, group_size=self.config.group_size,
                                     reduce_op="none" if r == 0 else "sum")
                if op == "mean":
                    ops.true_divide_(target, self.world_size)
        return self.reduced_shard(target, op=op, fused=fused, caller_owned=out is not None)

    def bound_reduce(self, received: torch.Tensor | None = None, *, op: str = "sum",
                     out: torch.Tensor | None = None) -> ops.BoundLaunch:
        """The fused launch of :meth:`reduce_received` (at most 8 ranks), bound and remembered but not issued."""
        if op not in ("sum", "mean"):
            raise ValueError(f"unsupported reduce-scatter mode: {op}")
        rows = self.received if received is None else received
        target = self.shard if out is None else out
        shard = self.chunks.shard_numel
        return self._remember(
            ("r", rows.data_ptr(), rows.numel(), target.data_ptr(), target.dtype, target.numel(), op),
            lambda: ops.bind_dequant_reduce(self._pairs(rows), target, numel=shard, group_size=self.config.group_size,
                                            divisor=float(self.world_size) if op == "mean" else 1.0))

    def reduced_shard(self, target: torch.Tensor, *, op: str, fused: bool = True, caller_owned: bool = False) -> ReducedShard:
        """The :class:`ReducedShard` record for this rank's shard held in ``target``."""
        shard = self.chunks.shard_numel
        metadata = {
            "compression_bit": self.config.bit, "group_size": self.config.group_size, "workspace_output": True,
            "workspace_shape": (shard,), "quantized_workspace_output": True, "received_workspace_output": True,
            "workspace_cache": True, "output_ownership": "caller" if caller_owned else "plan",
            "fused_dequant_reduce": fused, "chunk_plan_precompiled": True,
            "received_payload_numel": self.world_size * self.payload_bytes,
        }
        if not fused:
            metadata["fused_dequant_reduce_reason"] = (
                f"fused dequant supports at most {ops.MAX_PAYLOADS} input ranks; received {self.world_size}")
        return ReducedShard(shard=target, shard_index=self.rank, shard_numel=shard, original_shape=self.shape,
                            original_numel=self.numel, world_size=self.world_size, reduce=op,
                            padded_numel=self.chunks.padded_numel, dtype=ops.DTYPE_NAMES[self.reduced_dtype],
                            transport="compressed_all_to_all", metadata=metadata)

    def requantize_shard(self, shard: torch.Tensor | None = None) -> torch.Tensor:
        """Quantize the reduced shard into row ``rank`` of ``self.gathered``; returns that payload view."""
        source = self.shard if shard is None else shard
        row = self.payload(self.gathered, self.rank)

        def make() -> ops.BoundLaunch:
            codes, scales = ops.split_payload(row, self.chunks.shard_numel, self.config.group_size)
            return ops.bind_quant_pack(source, codes, scales, group_size=self.config.group_size)

        self._order_after_previous_use()
        bound = self._remember(("g", source.data_ptr(), source.dtype, source.numel()), make)
        if self.chunks.shard_numel and not bound():
            raise ValueError(f"no HIP quantize kernel for dtype {source.dtype}")
        return row

    def reduce_and_requantize(self, received: torch.Tensor | None = None, *, op: str = "sum") -> torch.Tensor:
        """The two steps above in one launch, for callers that only forward the requantized payload: row ``rank``
        of ``self.gathered`` receives ``quantize(reduce(received))`` and the full-precision shard is never written.
        Bit-identical to ``requantize_shard(reduce_received(...).shard)``.  Falls back to the two steps beyond 8
        ranks."""
        if op not in ("sum", "mean"):
            raise ValueError(f"unsupported reduce-scatter mode: {op}")
        rows = self.received if received is None else received
        row = self.payload(self.gathered, self.rank)
        shard = self.chunks.shard_numel
        if not shard:
            return row
        if self.world_size > ops.MAX_PAYLOADS:
            self.reduce_received(rows, op=op)
            return self.requantize_shard()
        self._order_after_previous_use()
        if not self.bound_reduce_requantize(rows, op=op)():
            raise ValueError(f"no HIP reduce-requantize kernel for dtype {self.reduced_dtype}")
        return row

    def bound_reduce_requantize(self, received: torch.Tensor | None = None, *, op: str = "sum") -> ops.BoundLaunch:
        """The launch of :meth:`reduce_and_requantize` (at most 8 ranks), bound and remembered but not issued."""
        if op not in ("sum", "mean"):
            raise ValueError(f"unsupported reduce-scatter mode: {op}")
        rows = self.received if received is None else received
        shard = self.chunks.shard_numel

        def make() -> ops.BoundLaunch:
            codes, scales = ops.split_payload(self.my_row, shard, self.config.group_size)
            return ops.bind_dequant_reduce_quant(self._pairs(rows), codes, scales, shard,
                                                 group_size=self.config.group_size,
                                                 divisor=float(self.world_size) if op == "mean" else 1.0,
                                                 mid_dtype=self.reduced_dtype)

        return self._remember(("rq", rows.data_ptr(), rows.numel(), op), make)

    def decode_gathered(self, gathered: torch.Tensor | None = None, *, out: torch.Tensor | None = None) -> torch.Tensor:
        """Decode the ``W`` gathered shard payloads into one flat tensor of the bucket's size (one launch)."""
        target = out if out is not None else torch.empty(self.numel, dtype=self.reduced_dtype, device=self.device)
        bound = self.bound_decode(target, gathered, remember=out is not None)
        self._order_after_previous_use()
        if self.numel and not bound():
            raise ValueError(f"no HIP decode kernel for dtype {target.dtype}")
        return target.reshape(self.shape)

    def bound_decode(self, target: torch.Tensor, gathered: torch.Tensor | None = None, *,
                     remember: bool = True) -> ops.BoundLaunch:
        """The launch of :meth:`decode_gathered` into ``target``, bound (and remembered, for a tensor that will come
        back) but not issued."""
        rows = self.gathered if gathered is None else gathered
        make = lambda: ops.bind_dequant_chunks(rows, target.reshape(-1), self.chunks.shard_numel,  # noqa: E731
                                               group_size=self.config.group_size)
        if not remember:
            return make()
        return self._remember(("d", rows.data_ptr(), rows.numel(), target.data_ptr(), target.dtype, target.numel()), make)


class AllGatherPlan(ReduceScatterPlan):
    """Pre-bound compute of one bucket shape for the all-gather form of the compressed all-reduce: every rank quantizes
    its whole bucket into one payload, the payloads are all-gathered, and one fused launch reduces the ``W`` of them in
    rank order into the bucket - the data path of the comm hook's ``all_gather`` strategy
    (``ccdl_comm/communication/ddp_hook.py:190-330``: quantize, gather, ``dequantize_reduce_tensors``) with its
    buffers and launches kept per bucket shape.  ``received`` is a matrix of ``W`` rows (everybody's payload) and
    ``send`` its row ``rank`` (this rank's); the inherited reduce steps read ``received`` and write ``numel`` elements."""

    def __init__(self, numel: int, dtype: torch.dtype, *, world_size: int, rank: int, config: CompressionConfig,
                 device: torch.device | str, reduced_dtype: torch.dtype | None = None,
                 shape: tuple[int, ...] | None = None) -> None:
        if config.bit != 8 or config.quant_type != "linear" or config.topk != 0 or config.stochastic:
            raise ValueError("the HIP all-gather plan supports linear 8-bit quantization without top-k / stochastic")
        if not 0 <= rank < world_size:
            raise ValueError(f"rank must be in [0, {world_size})")
        self.config = config
        self.world_size = world_size
        self.rank = rank
        self.numel = int(numel)
        self.shape = tuple(shape) if shape is not None else (self.numel,)
        self.dtype = dtype
        self.reduced_dtype = reduced_dtype or dtype
        self.device = torch.device(device)
        self.chunks = compile_chunk_plan(original_numel=self.numel, world_size=1)   # one chunk: the bucket
        self.payload_bytes = ops.payload_nbytes(self.numel, config.group_size)
        self.row_stride = -(-self.payload_bytes // _ROW_ALIGN) * _ROW_ALIGN
        self.received = torch.empty((world_size, self.row_stride), dtype=torch.uint8, device=self.device)
        # This rank's payload is quantized straight into its own row of the gather's output, the in-place form of an
        # all-gather (`dist.all_gather_into_tensor(received, received[rank])`): no copy of the local payload.
        self.send = self.received[rank:rank + 1]
        self.my_payload = self.received[rank, :self.payload_bytes]
        self._bound = OrderedDict()
        self._bound_lock = threading.Lock()
        self._last_stream = None
        self._last_stream_handle = None
        self.exchange_in_flight = None

    def bound_quantize(self, tensor: torch.Tensor, *, residual: torch.Tensor | None = None,
                       new_residual: torch.Tensor | None = None) -> ops.BoundLaunch:
        """The quantize + pack of the whole bucket (+ ``residual``) into ``self.send``, bound but not issued."""
        flat = tensor.reshape(-1)
        if flat.numel() != self.numel or flat.dtype != self.dtype:
            raise ValueError("tensor does not match the planned bucket")
        key = ("q", flat.data_ptr(), None if residual is None else (residual.data_ptr(), residual.dtype, residual.numel()),
               None if new_residual is None else (new_residual.data_ptr(), new_residual.dtype, new_residual.numel()))
        return self._remember(key, lambda: ops.bind_quant_pack_chunks(
            flat, self.send, 1, group_size=self.config.group_size,
            residual=None if residual is None else residual.reshape(-1),
            new_residual=None if new_residual is None else new_residual.reshape(-1)))

    def reduced_shard(self, target: torch.Tensor, *, op: str, fused: bool = True, caller_owned: bool = False) -> torch.Tensor:
        """What a bucket resolves to here: the reduced bucket itself, in the bucket's shape."""
        del op, fused, caller_owned
        return target.reshape(self.shape)

    def reduce_received(self, received: torch.Tensor | None = None, *, op: str = "sum",
                        out: torch.Tensor | None = None) -> torch.Tensor:
        if out is None:
            raise ValueError("the all-gather plan keeps no output buffer: pass out= (the bucket, or a tensor of its size)")
        return super().reduce_received(received, op=op, out=out)

    def bound_reduce(self, received: torch.Tensor | None = None, *, op: str = "sum",
                     out: torch.Tensor | None = None) -> ops.BoundLaunch:
        if out is None:
            raise ValueError("the all-gather plan keeps no output buffer: pass out= (the bucket, or a tensor of its size)")
        return super().bound_reduce(received, op=op, out=out)

    def _no_second_leg(self, *args: Any, **kwargs: Any) -> Any:
        raise TypeError("the all-gather form ends with the reduce of the gathered payloads: it has no requantize, "
                        "shard gather or decode step (those belong to ReduceScatterPlan)")

    requantize_shard = reduce_and_requantize = bound_reduce_requantize = decode_gathered = bound_decode = _no_second_leg

    def run(self, tensor: torch.Tensor, all_gather: Callable[[torch.Tensor, torch.Tensor], Any], *, op: str = "mean",
            out: torch.Tensor | None = None, residual: torch.Tensor | None = None) -> torch.Tensor:
        """The three steps one after the other: quantize, ``all_gather(received_rows, my_payload)``, fused reduce into
        ``out`` (default: a fresh tensor).  Beyond eight ranks the reduce decodes payload by payload."""
        target = out if out is not None else torch.empty(self.numel, dtype=self.reduced_dtype, device=self.device)
        self._order_after_previous_use()
        if self.numel and not self.bound_quantize(tensor, residual=residual, new_residual=residual)():
            raise ValueError(f"no HIP quantize kernel for dtype {tensor.dtype} with this residual")
        work = all_gather(self.received, self.my_payload)
        wait = getattr(work, "wait", None)
        if callable(wait):
            wait()
        return self.reduce_received(op=op, out=target.reshape(-1))


def compressed_reduce_scatter_shard(tensor: torch.Tensor, *, config: CompressionConfig, world_size: int, rank: int,
                                    all_to_all: Callable[[torch.Tensor, torch.Tensor], Any], op: str = "sum",
                                    plan: ReduceScatterPlan | None = None, async_op: bool = False,
                                    future_factory: Callable[[], Any] | None = None,
                                    completion_manager: Any | None = None,
                                    update_feedback: Callable[[ReducedShard], None] | None = None,
                                    advance_policy: Callable[[], None] | None = None, pipeline: Any | None = None,
                                    out: torch.Tensor | None = None) -> Any:
    """Quantize per-destination chunks, exchange, reduce: returns this rank's :class:`ReducedShard`.

    ``all_to_all(received_rows, send_rows)`` must fill row ``r`` of ``received_rows`` with rank ``r``'s
    payload for this rank (row ``rank`` of ``send_rows`` of that rank) - the one collective of the leg.

    ``async_op``: ``all_to_all`` starts the exchange and returns its work object (``wait()``, optionally
    ``get_future()``), e.g. ``dist.all_to_all_single(received, send, async_op=True)``; the call returns an
    :class:`~lowbit_comm_amd.communication.AsyncShardPipeline` that reduces the shard when the exchange is over
    and completes a future (``future_factory``, default ``torch.futures.Future``) with it
    (``ccdl_comm/communication/reduce_scatter_transport.py:286-333``).

    ``pipeline`` (with ``async_op``): a :class:`~lowbit_comm_amd.hip.bucket_pipeline.BucketPipeline` built without an
    all-gather, shared by the buckets of a stream.  The bucket's quantize then shares one launch with the reduce of the
    bucket handed over before it, and its own reduce goes out with the next bucket (or when the returned pipeline
    object is waited for, or at ``pipeline.flush()``); ``all_to_all``, ``world_size`` and ``rank`` are the pipeline's.
    ``out``: where this rank's shard is to be written (default: the plan's shard buffer, or a fresh tensor under a
    pipeline).
    """
    if pipeline is not None:
        if not async_op:
            raise ValueError("a bucket pipeline completes its buckets later: it needs async_op=True")
        return _shard_through_pipeline(tensor, config=config, op=op, pipeline=pipeline, out=out,
                                       future_factory=future_factory, completion_manager=completion_manager,
                                       update_feedback=update_feedback, advance_policy=advance_policy)
    if plan is None:
        plan = ReduceScatterPlan(tensor.numel(), tensor.dtype, world_size=world_size, rank=rank, config=config,
                                 device=tensor.device, shape=tuple(tensor.shape))
    send = plan.quantize_chunks(tensor)
    if not async_op:
        all_to_all(plan.received, send)
        return plan.reduce_received(op=op, out=out)
    from lowbit_comm_amd.communication.async_shard_pipeline import AsyncShardPipeline

    exchange = all_to_all(plan.received, send)
    if not callable(getattr(exchange, "wait", None)):
        raise TypeError("with async_op the exchange must return a work object with wait()")
    future = future_factory() if future_factory is not None else torch.futures.Future()
    plan.exchange_in_flight = exchange       # the exchange reads plan.send and writes plan.received on a stream of its own

    def reduce_shard(_received: Any) -> ReducedShard:   # runs once the exchange has been waited for
        plan.exchange_in_flight = None
        return plan.reduce_received(op=op, out=out)

    def release_plan(_done: Any) -> None:               # also when the exchange failed and the reduce never ran
        if plan.exchange_in_flight is exchange:
            plan.exchange_in_flight = None

    if callable(getattr(future, "add_done_callback", None)):
        future.add_done_callback(release_plan)

    return AsyncShardPipeline(communication_work=exchange, future=future, reduce_shard=reduce_shard,
                              update_feedback=update_feedback or (lambda _shard: None),
                              advance_policy=advance_policy or (lambda: None),
                              completion_manager=completion_manager, resources=(tensor, plan, send)).run()


class _ReduceEnqueued:
    """The 'exchange' an :class:`AsyncShardPipeline` sees for a bucket that went through a :class:`BucketPipeline`: it
    is over when the bucket's reduce has been enqueued, and what it delivers is the reduced shard itself."""

    def __init__(self, enqueued: Any) -> None:
        self._enqueued = enqueued

    def get_future(self) -> Any:
        return self._enqueued

    def wait(self) -> Any:
        return self._enqueued.wait()


def _shard_through_pipeline(tensor: torch.Tensor, *, config: CompressionConfig, op: str, pipeline: Any,
                            out: torch.Tensor | None, future_factory: Callable[[], Any] | None,
                            completion_manager: Any | None, update_feedback: Callable[[ReducedShard], None] | None,
                            advance_policy: Callable[[], None] | None) -> Any:
    from lowbit_comm_amd.communication.async_shard_pipeline import AsyncShardPipeline

    if pipeline.all_gather is not None:
        raise ValueError("the shard of a reduce-scatter comes from a pipeline built without all_gather")
    enqueued = pipeline.submit(tensor, config=config, op=op, out=out)
    # the outer future flushes the pipeline when somebody waits for it: the reduce of the stream's last bucket has no
    # later bucket to ride with
    outer = future_factory() if future_factory is not None else pipeline.make_future()
    return AsyncShardPipeline(communication_work=_ReduceEnqueued(enqueued), future=outer,
                              reduce_shard=lambda shard: shard,
                              update_feedback=update_feedback or (lambda _shard: None),
                              advance_policy=advance_policy or (lambda: None),
                              completion_manager=completion_manager, resources=(tensor, pipeline)).run()


def compressed_all_reduce_via_reduce_scatter(tensor: torch.Tensor, *, config: CompressionConfig, world_size: int,
                                             rank: int, all_to_all: Callable[[torch.Tensor, torch.Tensor], None],
                                             all_gather: Callable[[torch.Tensor, torch.Tensor], None],
                                             op: str = "sum", plan: ReduceScatterPlan | None = None,
                                             out: torch.Tensor | None = None, keep_shard: bool = False,
                                             residual: torch.Tensor | None = None) -> torch.Tensor:
    """Full plan: reduce-scatter leg, requantize, all-gather leg, decode every shard.

    ``residual`` (fp32 or the bucket's dtype, updated in place) turns on local error feedback in the quantize
    launch: the chunks encode ``tensor + residual`` and the residual becomes what that encoding dropped.

    Reduce and requantize run as one launch unless ``keep_shard`` asks for the full-precision shard in
    ``plan.shard`` as well.

    ``all_gather(gathered_rows, my_payload)`` must fill row ``r`` of ``gathered_rows`` with rank ``r``'s
    requantized shard payload (row ``rank`` is already in place).
    """
    if plan is None:
        plan = ReduceScatterPlan(tensor.numel(), tensor.dtype, world_size=world_size, rank=rank, config=config,
                                 device=tensor.device, shape=tuple(tensor.shape))
    if plan.numel == 0:       # nothing to exchange on any rank (reduce_scatter_transport.py:213-246 returns at once)
        return out.reshape(plan.shape) if out is not None else tensor
    if keep_shard:
        if residual is not None:
            raise ValueError("keep_shard and residual cannot be combined")
        compressed_reduce_scatter_shard(tensor, config=config, world_size=world_size, rank=rank,
                                        all_to_all=all_to_all, op=op, plan=plan)
        mine = plan.requantize_shard()
    else:
        send = plan.quantize_chunks(tensor, residual=residual, new_residual=residual)
        all_to_all(plan.received, send)
        mine = plan.reduce_and_requantize(op=op)
    all_gather(plan.gathered, mine)
    return plan.decode_gathered(out=out)


__all__ = ["AllGatherPlan", "ReduceScatterPlan", "ResidualStore", "compressed_all_reduce_async", "compressed_all_reduce_via_reduce_scatter",
           "compressed_reduce_scatter_shard", "make_all_gather_transport", "make_reduce_scatter_transport", "ccdl_dtype", "torch_dtype"]


def compressed_all_reduce_async(tensor: torch.Tensor, *, config: CompressionConfig, world_size: int, rank: int,
                                all_to_all: Callable[[torch.Tensor, torch.Tensor], None],
                                all_gather: Callable[[torch.Tensor, torch.Tensor], None], op: str = "sum",
                                plan: ReduceScatterPlan | None = None, out: torch.Tensor | None = None,
                                manager: Any | None = None, residual: torch.Tensor | None = None) -> Any:
    """:func:`compressed_all_reduce_via_reduce_scatter` on the communication stream: returns a work object at once.

    All four launches and the two exchanges are enqueued on a side stream ordered after the caller's current
    stream; ``work.wait()`` orders the caller's current stream after them (no host wait) and returns the reduced
    tensor.  The plan's workspaces and the input stay referenced by the work while it is in flight."""
    from lowbit_comm_amd.hip.completion import HipCompletionManager

    manager = manager if manager is not None else HipCompletionManager()
    if plan is None:
        plan = ReduceScatterPlan(tensor.numel(), tensor.dtype, world_size=world_size, rank=rank, config=config,
                                 device=tensor.device, shape=tuple(tensor.shape))
    stream_work = manager.create_stream_work(async_op=True)
    with stream_work:
        result = compressed_all_reduce_via_reduce_scatter(tensor, config=config, world_size=world_size, rank=rank,
                                                          all_to_all=all_to_all, all_gather=all_gather, op=op,
                                                          plan=plan, out=out, residual=residual)
        stream = getattr(stream_work, "stream", None)
        if stream is not None:            # the caching allocator must not reuse these before the side stream is done
            for held in (tensor, result) + (() if residual is None else (residual,)):
                held.record_stream(stream)
    return manager.create_work(result=result, completion=stream_work, resources=(tensor, plan, result, residual))


class ResidualStore(OrderedDict):
    """fp32 error-feedback residuals of a transport, one per bucket, keyed by the bucket's storage address, element
    count and dtype (a DDP bucket comes back at the same address every iteration).  Bounded: beyond ``max_entries`` the
    least recently used residual is dropped, and a bucket that returns after that starts from zero again - a caller
    that hands over fresh tensors every step would otherwise grow the store by one bucket-sized tensor per call."""

    def __init__(self, max_entries: int = 4096) -> None:
        super().__init__()
        if max_entries < 1:
            raise ValueError("max_entries must be at least 1")
        self.max_entries = max_entries

    def for_tensor(self, tensor: torch.Tensor) -> torch.Tensor:
        key = (tensor.data_ptr(), tensor.numel(), tensor.dtype)
        residual = self.get(key)
        if residual is None:
            residual = self[key] = torch.zeros(tensor.numel(), dtype=torch.float32, device=tensor.device)
            while len(self) > self.max_entries:
                self.popitem(last=False)
        else:
            self.move_to_end(key)
        return residual


def make_reduce_scatter_transport(*, world_size: int, rank: int,
                                  all_to_all: Callable[[torch.Tensor, torch.Tensor], None],
                                  all_gather: Callable[[torch.Tensor, torch.Tensor], None],
                                  max_plans: int = 64, manager: Any | None = None,
                                  inplace: bool = True, error_feedback: bool = False, pipelined: bool = False,
                                  lanes: int = 1, future_factory: Callable[[], Any] | None = None,
                                  max_residuals: int = 4096) -> Callable[..., Any]:
    """The callable ``create_ddp_comm_hook(reduce_scatter_all_gather=...)`` expects, over pre-bound plans.

    ``transport(tensor, *, config, op, async_op=False, dtype=None, extension_status=None)`` runs the compressed
    reduce-scatter + all-gather of ``tensor`` and returns the reduced tensor (``async_op``: a work object whose
    ``wait()`` returns it).  One :class:`ReduceScatterPlan` is kept per (element count, dtype, device, codec policy),
    so a bucket costs three pre-bound launches and the two injected exchanges from its second step on; the least
    recently used plan is dropped beyond ``max_plans``.  With ``inplace`` the decoded result overwrites ``tensor``
    (a DDP bucket is consumed by the quantize launch before the decode launch writes it), so nothing is allocated.
    With ``error_feedback`` every bucket (keyed by its storage address and size) keeps an fp32 residual that the
    quantize launch adds before encoding and refreshes with what the encoding dropped, in the same launch - the
    local error feedback of ``DDPBucketProcessor`` (``ccdl_comm/communication/ddp.py:69-97``); ``transport.residuals``
    exposes them (a :class:`ResidualStore`: the least recently used one is dropped beyond ``max_residuals``),
    ``transport.reset()`` drops them.  Counterpart of ``compressed_reduce_scatter_all_gather``
    (``ccdl_comm/communication/reduce_scatter_transport.py:186-377``) with the exchanges injected.

    ``pipelined``: the buckets go through a :class:`~lowbit_comm_amd.hip.bucket_pipeline.BucketPipeline` - one launch
    per bucket carries the quantize of that bucket, the reduce + requantize of the one before and the decode of the
    one before that; the transport then returns a future per bucket, ``transport.flush()`` issues what the last two
    buckets still wait for, and ``transport.pipelined`` is true (the comm hook flushes after the iteration's last
    bucket).  ``lanes`` deals the buckets to that many streams in turn.  More than eight ranks, and ``async_op``, take
    the unpipelined plan."""
    if pipelined and world_size <= ops.MAX_PAYLOADS:
        return _pipelined_transport(world_size=world_size, rank=rank, all_to_all=all_to_all, all_gather=all_gather,
                                    max_plans=max_plans, manager=manager, inplace=inplace, error_feedback=error_feedback,
                                    lanes=lanes, future_factory=future_factory, max_residuals=max_residuals)

    plans: OrderedDict = OrderedDict()
    residuals = ResidualStore(max_residuals)

    def residual_for(tensor: torch.Tensor) -> torch.Tensor | None:
        if not error_feedback or tensor.numel() == 0:
            return None
        return residuals.for_tensor(tensor)

    def plan_for(tensor: torch.Tensor, config: CompressionConfig) -> ReduceScatterPlan:
        key = (tensor.numel(), tensor.dtype, tensor.device, config.bit, config.group_size, config.topk,
               config.quant_type, config.stochastic)
        plan = plans.get(key)
        if plan is None:
            plan = plans[key] = ReduceScatterPlan(tensor.numel(), tensor.dtype, world_size=world_size, rank=rank,
                                                  config=config, device=tensor.device, shape=tuple(tensor.shape))
            while len(plans) > max_plans:
                plans.popitem(last=False)
        else:
            plans.move_to_end(key)
        return plan

    def transport(tensor: torch.Tensor, *, config: CompressionConfig, op: str = "sum", async_op: bool = False,
                  dtype: str | None = None, extension_status: Any | None = None) -> Any:
        del extension_status                      # the plan calls the C ABI directly
        if dtype is not None and torch_dtype(dtype) != tensor.dtype:
            raise ValueError(f"the reduce-scatter plan reduces in the bucket's dtype; got dtype={dtype!r} for {tensor.dtype}")
        plan = plan_for(tensor, config)
        out = tensor.reshape(-1) if inplace and tensor.is_contiguous() else None
        residual = residual_for(tensor)
        if async_op:
            return compressed_all_reduce_async(tensor, config=config, world_size=world_size, rank=rank,
                                               all_to_all=all_to_all, all_gather=all_gather, op=op, plan=plan,
                                               out=out, manager=manager, residual=residual)
        return compressed_all_reduce_via_reduce_scatter(tensor, config=config, world_size=world_size, rank=rank,
                                                        all_to_all=all_to_all, all_gather=all_gather, op=op, plan=plan,
                                                        out=out, residual=residual)

    transport.plans = plans
    transport.residuals = residuals
    transport.reset = residuals.clear
    transport.pipelined = False
    transport.flush = lambda: None
    return transport


def make_all_gather_transport(*, world_size: int, rank: int, all_gather: Callable[[torch.Tensor, torch.Tensor], Any],
                              max_plans: int = 64, inplace: bool = True, error_feedback: bool = False,
                              pipelined: bool = False, lanes: int = 1, future_factory: Callable[[], Any] | None = None,
                              max_residuals: int = 4096) -> Callable[..., Any]:
    """A whole-collective transport for ``create_ddp_comm_hook`` (``strategy="topology"`` with
    ``topology_all_reduce=``, or any other strategy that takes one) that runs the all-gather form of the compressed
    all-reduce - the data path of the hook's own ``all_gather`` strategy (``ccdl_comm/communication/ddp_hook.py:190-330``:
    quantize, all-gather of the payloads, fused dequantize-reduce) - over pre-bound :class:`AllGatherPlan` objects.

    ``all_gather(received_rows, my_payload)`` fills row ``r`` of ``received_rows`` with rank ``r``'s payload;
    ``my_payload`` already lies in row ``rank`` (the in-place form: ``dist.all_gather_into_tensor(received_rows,
    received_rows[rank])``); it may return a work object.  ``transport(tensor, *, config, op,
    async_op=False, dtype=None, extension_status=None)`` reduces ``tensor`` - in place with ``inplace`` - and returns it.

    ``pipelined``: buckets go through a :class:`~lowbit_comm_amd.hip.bucket_pipeline.BucketPipeline`; the
    quantize of bucket k shares one launch with the reduce of bucket k-1 (``lbc_quant_pack_chunks_and_dequant_reduce``),
    the transport returns a future per bucket, ``transport.flush()`` issues the last reduce and ``transport.pipelined``
    is true, so the comm hook flushes after the iteration's last bucket.  ``error_feedback`` keeps an fp32 residual per
    bucket (local error feedback, fused into the quantize launch; at most ``max_residuals`` of them).  More than eight
    ranks take the unpipelined plan, whose reduce then decodes payload by payload.  The form is bound by its reduce,
    which reads ``W`` payloads: pipelining saves host time (14 against 17 us per 25 MiB bf16 bucket; 24 us through the
    codec facade), not GPU time (33-35 us either way at W = 8)."""
    residuals = ResidualStore(max_residuals)
    plans: OrderedDict[Any, AllGatherPlan] = OrderedDict()
    lock = threading.Lock()

    def plan_for(tensor: torch.Tensor, config: CompressionConfig) -> AllGatherPlan:
        key = (tensor.numel(), tensor.dtype, tensor.device, config.bit, config.group_size, config.topk, config.quant_type,
               config.stochastic)
        with lock:
            plan = plans.get(key)
            if plan is None:
                plan = plans[key] = AllGatherPlan(tensor.numel(), tensor.dtype, world_size=world_size, rank=rank, config=config,
                                                  device=tensor.device, shape=tuple(tensor.shape))
                while len(plans) > max_plans:
                    plans.popitem(last=False)
            else:
                plans.move_to_end(key)
        return plan

    def unpipelined(tensor: torch.Tensor, config: CompressionConfig, op: str) -> torch.Tensor:
        if tensor.numel() == 0:
            return tensor
        in_place = inplace and tensor.is_contiguous()
        residual = residuals.for_tensor(tensor) if error_feedback else None
        reduced = plan_for(tensor, config).run(tensor, all_gather, op=op, out=tensor.reshape(-1) if in_place else None,
                                               residual=residual)
        return reduced.reshape(tensor.shape)

    pipeline = None
    if pipelined and world_size <= ops.MAX_PAYLOADS:
        from lowbit_comm_amd.hip.bucket_pipeline import BucketPipeline

        pipeline = BucketPipeline(world_size=world_size, rank=rank, whole_gather=all_gather, error_feedback=error_feedback,
                                  inplace=inplace, lanes=lanes, max_plans=max_plans, future_factory=future_factory,
                                  max_residuals=max_residuals)
        residuals = pipeline.residuals

    def transport(tensor: torch.Tensor, *, config: CompressionConfig, op: str = "sum", async_op: bool = False,
                  dtype: str | None = None, extension_status: Any | None = None) -> Any:
        del extension_status                      # the plans call the C ABI directly
        if op not in ("sum", "mean"):
            raise ValueError(f"unsupported all-reduce mode: {op}")
        if dtype is not None and torch_dtype(dtype) != tensor.dtype:
            raise ValueError(f"the all-gather plan reduces in the bucket's dtype; got dtype={dtype!r} for {tensor.dtype}")
        if async_op:
            from lowbit_comm_amd.work import ImmediateWork

            if pipeline is not None:
                pipeline.flush()                  # a work object promises a result to whoever waits: nothing is held back
            return ImmediateWork(unpipelined(tensor, config, op))
        if pipeline is not None:
            return pipeline.submit(tensor, config=config, op=op)
        return unpipelined(tensor, config, op)

    transport.pipeline = pipeline
    transport.plans = plans if pipeline is None else pipeline._plans
    transport.residuals = residuals
    transport.pipelined = pipeline is not None
    if pipeline is not None:
        transport.flush = pipeline.flush
        transport.reset = pipeline.reset
    else:
        transport.reset = residuals.clear
    return transport


def _pipelined_transport(*, world_size: int, rank: int, all_to_all: Callable[..., Any], all_gather: Callable[..., Any],
                         max_plans: int, manager: Any | None, inplace: bool, error_feedback: bool, lanes: int,
                         future_factory: Callable[[], Any] | None, max_residuals: int) -> Callable[..., Any]:
    from lowbit_comm_amd.hip.bucket_pipeline import BucketPipeline

    pipeline = BucketPipeline(world_size=world_size, rank=rank, all_to_all=all_to_all, all_gather=all_gather,
                              error_feedback=error_feedback, inplace=inplace, lanes=lanes, max_plans=max_plans,
                              future_factory=future_factory, max_residuals=max_residuals)
    unpipelined = make_reduce_scatter_transport(world_size=world_size, rank=rank, all_to_all=all_to_all,
                                                all_gather=all_gather, max_plans=max_plans, manager=manager,
                                                inplace=inplace, error_feedback=False)

    def transport(tensor: torch.Tensor, *, config: CompressionConfig, op: str = "sum", async_op: bool = False,
                  dtype: str | None = None, extension_status: Any | None = None) -> Any:
        del extension_status                      # the plans call the C ABI directly
        if dtype is not None and torch_dtype(dtype) != tensor.dtype:
            raise ValueError(f"the reduce-scatter plan reduces in the bucket's dtype; got dtype={dtype!r} for {tensor.dtype}")
        if async_op:
            if error_feedback:
                raise ValueError("the pipelined transport keeps the residuals; async_op is served by the unpipelined plan, "
                                 "which would not see them")
            pipeline.flush()
            return unpipelined(tensor, config=config, op=op, async_op=True)
        return pipeline.submit(tensor, config=config, op=op)

    transport.pipeline = pipeline
    transport.plans = pipeline._plans
    transport.residuals = pipeline.residuals
    transport.reset = pipeline.reset
    transport.pipelined = True
    transport.flush = pipeline.flush
    return transport
