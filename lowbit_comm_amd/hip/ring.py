"""Quantized ring all-reduce: compiled per-rank schedule, executor and the gfx950 runtime of its compute steps.

Counterparts in the reference: the schedule types and ``compile_pipelined_ring_schedule``
(``ccdl_comm/cuda/transports/pipelined_ring.py:19-110,285-331``), ``PipelinedRingExecutor`` (``:174-282``) with the
ownership rules of ``ccdl_comm/cuda/transports/_executor_support.py``, and ``TorchPipelinedRingRuntime``
(``ccdl_comm/cuda/transports/torch_topology.py:67-316``).

A ring over W ranks moves every chunk of the bucket W-1 hops while it is summed (reduce-scatter) and W-1 hops while
the mean is handed round (all-gather).  One rule generates the whole schedule: a rank always sends the chunk it has
just received into, starting with its predecessor's chunk index, so that after W-1 steps rank r holds the complete
chunk r.  The reference runs "decode into the chunk" and "quantize the chunk for the next hop" as separate kernels;
the runtime here issues them as one launch of the ring-step kernel (``lbc_ring_step``), which quantizes the updated
chunk while it is still in registers, and hands the staged payload to the next ``quant_pack`` call.  The point-to-point
exchange itself is injected: ``exchange(payload, received, send_peer=, recv_peer=, stream=) -> handle``.
"""
from __future__ import annotations

import threading
from dataclasses import dataclass, field
from typing import Any, Callable

from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.hip.chunk_plan import ChunkPlan, ChunkRange, compile_chunk_plan

# --------------------------------------------------------------------------- #
# schedule
# --------------------------------------------------------------------------- #
_STEP_INTEGERS = ("step_index", "send_peer", "recv_peer", "send_chunk_owner", "recv_chunk_owner")


def _natural(value: object, name: str) -> None:
    if isinstance(value, bool) or not isinstance(value, int):
        raise TypeError(f"{name} must be an integer")
    if value < 0:
        raise ValueError(f"{name} must be >= 0")


def _rank_of(value: object, world_size: int, name: str) -> None:
    _natural(value, name)
    if value >= world_size:
        raise ValueError(f"{name} must be in [0, {world_size})")


def _check_step(step: Any) -> None:
    for name in _STEP_INTEGERS:
        _natural(getattr(step, name), name)
    for name in ("send_chunk", "recv_chunk"):
        if not isinstance(getattr(step, name), ChunkRange):
            raise TypeError(f"{name} must be a ChunkRange")


@dataclass(frozen=True)
class RingReduceScatterStep:
    """One hop of the summing phase.  ``received_contributors``: the ranks whose data the arriving payload already
    sums, oldest first; its length is ``step_index + 1``."""

    step_index: int
    send_peer: int
    recv_peer: int
    send_chunk_owner: int
    recv_chunk_owner: int
    received_contributors: tuple[int, ...]
    send_chunk: ChunkRange
    recv_chunk: ChunkRange

    def __post_init__(self) -> None:
        _check_step(self)
        ranks = self.received_contributors
        if not isinstance(ranks, tuple):
            raise TypeError("received_contributors must be a tuple")
        if not ranks:
            raise ValueError("received_contributors must not be empty")
        for entry in ranks:
            _natural(entry, "received_contributors entry")
        if len(set(ranks)) != len(ranks):
            raise ValueError("received_contributors must not contain duplicates")
        if len(ranks) != self.step_index + 1:
            raise ValueError("received_contributors length must equal step_index + 1")


@dataclass(frozen=True)
class RingAllGatherStep:
    """One hop of the phase that hands the reduced chunks round."""

    step_index: int
    send_peer: int
    recv_peer: int
    send_chunk_owner: int
    recv_chunk_owner: int
    send_chunk: ChunkRange
    recv_chunk: ChunkRange

    def __post_init__(self) -> None:
        _check_step(self)


def _hops(world_size: int, first_sent: int):
    """``(step, sent chunk, received chunk)``: what is received is what the predecessor sent, one index lower,
    and it is what goes out next."""
    sent = first_sent
    for step in range(world_size - 1):
        received = (sent - 1) % world_size
        yield step, sent, received
        sent = received


def _reduce_steps(plan: ChunkPlan, rank: int) -> tuple[RingReduceScatterStep, ...]:
    world = plan.world_size
    after, before = (rank + 1) % world, (rank - 1) % world
    return tuple(
        RingReduceScatterStep(step_index=step, send_peer=after, recv_peer=before, send_chunk_owner=sent,
                              recv_chunk_owner=received,
                              received_contributors=tuple((before - back) % world for back in range(step, -1, -1)),
                              send_chunk=plan.chunk_for_rank(sent), recv_chunk=plan.chunk_for_rank(received))
        for step, sent, received in _hops(world, before))


def _gather_steps(plan: ChunkPlan, rank: int) -> tuple[RingAllGatherStep, ...]:
    world = plan.world_size
    after, before = (rank + 1) % world, (rank - 1) % world
    return tuple(
        RingAllGatherStep(step_index=step, send_peer=after, recv_peer=before, send_chunk_owner=sent,
                          recv_chunk_owner=received, send_chunk=plan.chunk_for_rank(sent),
                          recv_chunk=plan.chunk_for_rank(received))
        for step, sent, received in _hops(world, rank))


@dataclass(frozen=True)
class PipelinedRingSchedule:
    """The steps of one rank, bound to an immutable chunk plan; only the deterministic schedule is accepted."""

    chunk_plan: ChunkPlan
    rank: int
    steps: tuple[RingReduceScatterStep, ...]
    gather_steps: tuple[RingAllGatherStep, ...]

    def __post_init__(self) -> None:
        if not isinstance(self.chunk_plan, ChunkPlan):
            raise TypeError("chunk_plan must be a ChunkPlan")
        _rank_of(self.rank, self.chunk_plan.world_size, "rank")
        if self.steps != _reduce_steps(self.chunk_plan, self.rank):
            raise ValueError("steps must match the deterministic ring schedule")
        if self.gather_steps != _gather_steps(self.chunk_plan, self.rank):
            raise ValueError("gather_steps must match the deterministic ring schedule")

    @property
    def local_chunk(self) -> ChunkRange:
        """The chunk this rank holds completely reduced after the first phase."""
        return self.chunk_plan.chunk_for_rank(self.rank)


def compile_pipelined_ring_schedule(*, chunk_plan: ChunkPlan, rank: int) -> PipelinedRingSchedule:
    if not isinstance(chunk_plan, ChunkPlan):
        raise TypeError("chunk_plan must be a ChunkPlan")
    _rank_of(rank, chunk_plan.world_size, "rank")
    return PipelinedRingSchedule(chunk_plan=chunk_plan, rank=rank, steps=_reduce_steps(chunk_plan, rank),
                                 gather_steps=_gather_steps(chunk_plan, rank))


# --------------------------------------------------------------------------- #
# completion plumbing shared by the executor
# --------------------------------------------------------------------------- #
def _probe(value: Any) -> Callable[[], Any] | None:
    for name in ("query", "is_completed"):
        method = getattr(value, name, None)
        if callable(method):
            return method
    return None


def _require_endpoint(value: Any, name: str) -> None:
    if _probe(value) is None:
        raise TypeError(f"{name} must provide nonblocking query() or is_completed()")
    for method in ("wait", "wait_stream"):
        if not callable(getattr(value, method, None)):
            raise TypeError(f"{name} must provide {method}()")


@dataclass(frozen=True)
class JoinedCompletion:
    """Ready when the submission context (the producer of the tensor) and the runtime's recorded end both are."""

    context: Any
    runtime_completion: Any

    def __post_init__(self) -> None:
        _require_endpoint(self.context, "submission context")
        _require_endpoint(self.runtime_completion, "runtime completion")

    def query(self) -> bool:
        return bool(_probe(self.context)()) and bool(_probe(self.runtime_completion)())

    def is_completed(self) -> bool:
        return self.query()

    def wait(self) -> None:
        self.context.wait()
        self.runtime_completion.wait()

    def wait_stream(self, stream: Any) -> None:
        self.context.wait_stream(stream)
        self.runtime_completion.wait_stream(stream)


@dataclass(eq=False)
class _Submission:
    """Everything one ``run()`` holds on to until the device has finished with it."""

    tensor: Any
    workspace: Any
    context: Any
    resources: list = field(default_factory=list)
    dependencies: list = field(default_factory=list)
    completion: Any = None
    record_attempted: bool = False
    failed: bool = False
    settled: bool = False          # workspace released or aborted

    def __post_init__(self) -> None:
        self.resources += [self.tensor, self.workspace, self.context]

    def keep(self, *values: Any) -> None:
        self.resources += [v for v in values if v is not None]

    def after(self, value: Any) -> None:
        if value is not None:
            self.dependencies.append(value)
            self.keep(value)

    def after_p2p(self, value: Any) -> None:
        self.keep(value)
        if _probe(value) is None:
            raise TypeError("P2P dependency must provide nonblocking query() or is_completed()")
        self.dependencies.append(value)

    def keep_workspace_buffers(self) -> None:
        leases = getattr(self.workspace, "leases", ())
        if isinstance(leases, tuple):
            self.keep(*leases)


class TopologyExecutor:
    """Enqueues the whole schedule of one rank without waiting on the host and returns completion-backed work.

    ``workspace_session_factory(tensor)`` gives a session with ``release(completion=)`` and optionally ``abort()``;
    ``completion_manager.create_work(result=, completion=, resources=)`` the work object.  A submission that fails
    after device work was enqueued keeps its buffers until that work has drained (``reap_pending``), then aborts
    the session instead of releasing it (the ownership rules of
    ``ccdl_comm/cuda/transports/_executor_support.py:121-257``).  Subclasses say what a schedule is and enqueue its
    steps in :meth:`_enqueue`."""

    schedule_type: type = object

    def __init__(self, *, schedule: Any, runtime: Any, workspace_session_factory: Callable[[Any], Any],
                 completion_manager: Any) -> None:
        if not isinstance(schedule, self.schedule_type):
            raise TypeError(f"schedule must be a {self.schedule_type.__name__}")
        if not callable(workspace_session_factory):
            raise TypeError("workspace_session_factory must be callable")
        self.schedule = schedule
        self._runtime = runtime
        self._sessions = workspace_session_factory
        self._works = completion_manager
        self._pending: list[_Submission] = []
        self._busy = threading.Lock()

    @property
    def pending_submission_count(self) -> int:
        return len(self._pending)

    def reap_pending(self) -> None:
        if not self._busy.acquire(blocking=False):
            raise RuntimeError("cannot reap while topology submission is in progress")
        try:
            self._reap()
        finally:
            self._busy.release()

    def run(self, tensor: Any) -> Any:
        if not self._busy.acquire(blocking=False):
            raise RuntimeError("concurrent run() on one topology executor is unsupported")
        try:
            return self._submit(tensor)
        finally:
            self._busy.release()

    # ---- one submission ---------------------------------------------------- #
    def _submit(self, tensor: Any) -> Any:
        self._reap()
        runtime = self._runtime
        context = runtime.create_submission_context(tensor)
        _require_endpoint(context, "submission context")
        submission = _Submission(tensor=tensor, workspace=self._sessions(tensor), context=context)
        try:
            runtime.wait_for_producer(tensor, context=context)
            self._enqueue(submission)
            self._record(submission)
            return self._finish(submission)
        except BaseException:
            self._fail(submission)
            raise

    def _enqueue(self, submission: _Submission) -> None:
        raise NotImplementedError

    def _record(self, submission: _Submission) -> None:
        submission.record_attempted = True
        ended = self._runtime.record_completion(context=submission.context,
                                                dependencies=tuple(submission.dependencies))
        submission.keep(ended)
        submission.completion = JoinedCompletion(submission.context, ended)
        submission.keep(submission.completion)

    def _finish(self, submission: _Submission) -> Any:
        submission.keep_workspace_buffers()
        self._hold(submission)
        work = self._works.create_work(result=submission.tensor, completion=submission.completion,
                                       resources=tuple(submission.resources))
        submission.keep(work)
        self._release(submission, submission.completion)
        self._pending.remove(submission)
        return work

    def _fail(self, submission: _Submission) -> None:
        submission.failed = True
        submission.keep_workspace_buffers()
        self._hold(submission)
        if not submission.record_attempted:
            try:
                self._record(submission)      # so that there is something to wait for before the buffers go back
            except BaseException:
                pass

    def _hold(self, submission: _Submission) -> None:
        if submission not in self._pending:
            self._pending.append(submission)

    @staticmethod
    def _release(submission: _Submission, completion: Any) -> None:
        release = getattr(submission.workspace, "release", None)
        if not callable(release):
            raise TypeError("workspace session must provide release(completion=...)")
        release(completion=completion)
        submission.settled = True

    def _reap(self) -> None:
        for submission in tuple(self._pending):
            readiness = submission.completion if submission.completion is not None else submission.context
            probe = _probe(readiness)
            try:
                if probe is None or not probe():
                    continue
            except BaseException:
                continue
            if not submission.settled:
                abort = getattr(submission.workspace, "abort", None)
                try:
                    if submission.failed and callable(abort):
                        abort()
                        submission.settled = True
                    else:
                        self._release(submission, readiness)
                except BaseException:
                    continue
            self._pending.remove(submission)


class PipelinedRingExecutor(TopologyExecutor):
    """The ring: per hop ``quant_pack``, ``send_recv``, then ``fused_reduce`` (first phase) or ``apply_broadcast``
    (second phase) - the runtime protocol and call order of ``ccdl_comm/cuda/transports/pipelined_ring.py:113-275``."""

    schedule_type = PipelinedRingSchedule

    def _enqueue(self, submission: _Submission) -> None:
        runtime, tensor, context, workspace = self._runtime, submission.tensor, submission.context, submission.workspace
        replay = getattr(runtime, "replay_program", None)
        if callable(replay):
            handles = replay(context)
            if handles is not None:          # this tensor's launches and exchanges were recorded by an earlier run
                for handle in handles:
                    submission.after_p2p(handle)
                return
        for step in self.schedule.steps:
            received, handle = self._exchange(submission, step)
            submission.after(runtime.fused_reduce(tensor, received, step.recv_chunk, step.received_contributors,
                                                  workspace, context=context, dependency=handle))
        for step in self.schedule.gather_steps:
            received, handle = self._exchange(submission, step)
            submission.after(runtime.apply_broadcast(tensor, received, step.recv_chunk, workspace,
                                                     context=context, dependency=handle))
        finish = getattr(runtime, "finish_program", None)
        if callable(finish):
            finish(context)

    def _exchange(self, submission: _Submission, step: Any) -> tuple[Any, Any]:
        runtime, context, workspace = self._runtime, submission.context, submission.workspace
        payload = runtime.quant_pack(submission.tensor, step.send_chunk, workspace, context=context)
        submission.keep(payload)
        received, handle = runtime.send_recv(payload, send_peer=step.send_peer, recv_peer=step.recv_peer,
                                             recv_chunk=step.recv_chunk, workspace=workspace, context=context)
        submission.keep(received)
        submission.after_p2p(handle)
        return received, handle


# --------------------------------------------------------------------------- #
# gfx950 runtime of the compute steps
# --------------------------------------------------------------------------- #
@dataclass
class RingSubmissionContext:
    """Per-submission state; nothing mutable is shared between runs."""

    tensor: Any
    stream: Any
    producer_completion: Any
    quant_index: int = 0
    recv_index: int = 0
    mean_applied: bool = False
    steps_done: int = 0
    staged: tuple | None = None        # ((start, stop), payload) quantized by the previous step's launch
    plan: dict | None = None           # buffers and bound launches of this tensor, when the runtime keeps plans
    raw_stream: int = 0
    program: list | None = None        # the launches and exchanges of this run in order, while a plan is being made

    def query(self) -> bool:
        return bool(self.producer_completion.query())

    def wait(self) -> None:
        self.producer_completion.wait()

    def wait_stream(self, stream: Any) -> None:
        self.producer_completion.wait_stream(stream)


def _view(tensor: Any, chunk: ChunkRange) -> Any:
    return tensor.reshape((-1,))[chunk.start:chunk.stop]


class HipPipelinedRingRuntime:
    """The coarse operations of the ring on one gfx950 device, for the portable INT8 payload
    ``uint8[codes || fp32 scales]``.

    ``fuse_steps=True`` (default): ``fused_reduce`` / ``apply_broadcast`` run the ring-step kernel, which also
    quantizes the updated chunk into the send buffer of the next step; the following ``quant_pack`` of that chunk
    returns the staged payload without a launch.  ``fuse_steps=False`` issues the reference's sequence (decode with
    reduce op, in-place division, quantize) as separate launches; both give the same bits.  Unlike the reference's
    native path, chunks need not be multiples of the group size.

    ``max_plans > 0`` (default 16): the send and receive buffers of a bucket and its validated, marshalled launches
    are kept per ``(address, numel)`` of the tensor and replayed on later runs, least recently used plans dropped
    first; the workspace session is then not asked for buffers.  One plan holds ``4 (W - 1)`` payload buffers.  All of
    a runtime's work is enqueued on its one stream, which orders the reuse of those buffers between runs.
    ``max_plans=0``: every run leases its buffers from the workspace session.

    With plans, the first run on a tensor also records its launches and exchanges in order, and later runs replay that
    list without going through the per-hop protocol again (14 hops of a W=8 ring: 193 us of host time per bucket
    through the protocol, which left the GPU waiting; the replay is a loop over pre-bound calls).
    ``graph_replay=True``: the second run captures the list as one HIP graph - the injected ``exchange`` must then
    be capturable on the stream it is given (enqueue-only, no host synchronisation, no allocation) - and later runs
    replay the graph.  Results are the same bits either way.

    ``extension_status``: run the steps through the codec facade of that native module instead
    (``quantize_tensor(view, output=...)``, ``dequantize_tensor(received, output=view, reduce_op=...)``,
    ``view.div_(W)``), exactly the calls of the reference's runtime.  This serves every policy and payload format
    the module does - in particular the CUDA extension's byte format, for rings that mix ranks running that
    extension with gfx950 ranks - at the reference's launch count; chunks must then be whole groups, as there.
    Plain linear 8-bit codes in the CUDA byte format do not need the facade: with ``fuse_steps`` they take that
    format's own fused step (``lbc_wire_ring_step``), one launch per hop as in the portable format."""

    def __init__(self, *, config: CompressionConfig, dtype: str, world_size: int, rank: int,
                 exchange: Callable[..., Any], completion_manager: Any | None = None, stream: Any | None = None,
                 fuse_steps: bool = True, max_plans: int = 16, extension_status: Any | None = None,
                 graph_replay: bool = False) -> None:
        from collections import OrderedDict

        from lowbit_comm_amd.hip.executors import fused_dequant_fallback_reason

        reason = None if extension_status is not None else fused_dequant_fallback_reason(config)
        if reason is not None:
            raise ValueError(reason.replace("fused dequant", "the ring runtime"))
        if dtype not in ("fp32", "fp16", "bf16"):
            raise ValueError(f"unsupported dtype {dtype!r}")
        if isinstance(world_size, bool) or not isinstance(world_size, int) or world_size <= 0:
            raise ValueError("world_size must be a positive integer")
        _rank_of(rank, world_size, "rank")
        if not callable(exchange):
            raise TypeError("exchange must be callable")
        if isinstance(max_plans, bool) or not isinstance(max_plans, int) or max_plans < 0:
            raise ValueError("max_plans must be an integer >= 0")
        self.config = config
        self.dtype = dtype
        self.world_size = world_size
        self.rank = rank
        module = getattr(extension_status, "module", None)
        cuda_bytes = extension_status is not None and getattr(module, "NATIVE_WIRE_FORMAT", "native") == "native"
        plain = config.bit == 8 and config.quant_type == "linear" and config.topk == 0 and not config.stochastic
        # the CUDA byte format has a fused step of its own for plain linear 8-bit codes; everything else a module
        # serves goes through its facade
        self._wire_direct = bool(fuse_steps) and cuda_bytes and plain
        self._facade = extension_status is not None and not self._wire_direct
        self.fuse_steps = bool(fuse_steps) and not self._facade
        self.extension_status = extension_status
        self.max_plans = max_plans
        self.plans: "OrderedDict[tuple[int, int], dict]" = OrderedDict()
        self._exchange = exchange
        self._completions = completion_manager
        self.stream = stream
        self.graph_replay = bool(graph_replay)

    # ---- context ----------------------------------------------------------- #
    def _ready(self) -> None:
        import torch

        if self._completions is None:
            from lowbit_comm_amd.hip.completion import HipCompletionManager

            self._completions = HipCompletionManager()
        if self.stream is None:
            self.stream = torch.cuda.Stream()       # default priority

    def _plan_of(self, tensor: Any) -> dict | None:
        if self.max_plans == 0:
            return None
        key = (tensor.data_ptr(), tensor.numel())
        plan = self.plans.get(key)
        if plan is None:
            while len(self.plans) >= self.max_plans:
                self.plans.popitem(last=False)
            plan = self.plans[key] = {}
        else:
            self.plans.move_to_end(key)
        return plan

    def create_submission_context(self, tensor: Any) -> RingSubmissionContext:
        import torch

        from lowbit_comm_amd.hip import ops

        self._ready()
        if not isinstance(tensor, torch.Tensor) or not tensor.is_cuda or not tensor.is_contiguous():
            raise RuntimeError("the ring runs in place on a contiguous GPU tensor")
        if ops.DTYPE_NAMES.get(tensor.dtype) != self.dtype:
            raise RuntimeError(f"tensor dtype {tensor.dtype} does not match the runtime's {self.dtype}")
        from lowbit_comm_amd.hip.workspace import StreamOrderedCompletion

        # The producer's work so far: no event unless the ring runs on another stream than the producer.
        produced = StreamOrderedCompletion(torch.cuda.current_stream(tensor.device))
        plan = self._plan_of(tensor)
        recording = plan is not None and "program" not in plan and not self._facade
        return RingSubmissionContext(tensor=tensor, stream=self.stream, producer_completion=produced,
                                     plan=plan, raw_stream=self.stream.cuda_stream, program=[] if recording else None)

    # ---- replay of a recorded run ------------------------------------------- #
    def finish_program(self, context: RingSubmissionContext) -> None:
        """The schedule has been enqueued once through the protocol: keep what it launched, in order."""
        if context.plan is not None and context.program is not None:
            context.plan["program"] = tuple(context.program)
            context.program = None

    def _run_program(self, program: tuple, stream: Any, raw_stream: int) -> list:
        handles = []
        for op in program:
            kind = op[0]
            if kind == "launch":
                if not op[1](raw_stream):
                    raise RuntimeError("a ring launch has no kernel for this configuration")
            elif kind == "exchange":
                handle = self._exchange(op[1], op[2], send_peer=op[3], recv_peer=op[4], stream=stream)
                handle.wait_stream(stream)
                handles.append(handle)
            else:                                    # "divide": the unfused sequence's in-place mean
                import torch

                from lowbit_comm_amd.hip import ops

                with torch.cuda.stream(stream):
                    ops.true_divide_(op[1], op[2])
        return handles

    def replay_program(self, context: RingSubmissionContext) -> list | None:
        """Enqueue the recorded launches and exchanges of this tensor's plan; ``None`` when there is no record yet."""
        plan = context.plan
        program = None if plan is None else plan.get("program")
        if program is None:
            return None
        if not self.graph_replay:
            return self._run_program(program, context.stream, context.raw_stream)
        import torch

        graph = plan.get("graph")
        if graph is None:
            graph = torch.cuda.CUDAGraph()
            side = torch.cuda.Stream()               # default priority; capture needs a stream of its own
            side.wait_stream(context.stream)
            with torch.cuda.graph(graph, stream=side):
                self._run_program(program, side, side.cuda_stream)
            context.stream.wait_stream(side)
            plan["graph"] = graph
        with torch.cuda.stream(context.stream):
            graph.replay()
        return []

    def wait_for_producer(self, tensor: Any, *, context: RingSubmissionContext) -> None:
        context.wait_stream(context.stream)
        tensor.record_stream(context.stream)

    def record_completion(self, *, context: RingSubmissionContext, dependencies: tuple[Any, ...]) -> Any:
        for dependency in dependencies:
            wait_stream = getattr(dependency, "wait_stream", None)
            if callable(wait_stream):
                wait_stream(context.stream)
        import torch

        from lowbit_comm_amd.hip.workspace import StreamOrderedCompletion

        if context.stream == torch.cuda.current_stream(context.tensor.device):
            return StreamOrderedCompletion(context.stream)     # the caller's own stream: its order is the completion
        return self._completions.record_for(context.tensor, stream=context.stream)

    # ---- buffers ----------------------------------------------------------- #
    def _payload_nbytes(self, numel: int) -> int:
        from lowbit_comm_amd.quantization.sizing import estimate_quantized_size

        wire = "portable"
        if self.extension_status is not None:
            wire = getattr(getattr(self.extension_status, "module", None), "NATIVE_WIRE_FORMAT", "native")
        return estimate_quantized_size(numel, dtype=self.dtype, config=self.config, wire_format=wire).quantized_bytes

    def _payload_buffer(self, kind: str, index: int, view: Any, workspace: Any, context: RingSubmissionContext) -> Any:
        """Send or receive buffer number ``index`` of this submission, sized for ``view``'s chunk."""
        plan = context.plan
        if plan is not None or self.extension_status is not None:      # the pool sizes portable payloads only
            buffer = None if plan is None else plan.get((kind, index))
            if buffer is None:
                import torch

                with torch.cuda.stream(context.stream):
                    buffer = torch.empty(self._payload_nbytes(view.numel()), dtype=torch.uint8, device=view.device)
                if plan is not None:
                    plan[(kind, index)] = buffer
            return buffer
        if kind == "send":
            return workspace.get_quantized_chunk(id(context.tensor), index, view, self.config, dtype=self.dtype,
                                                 world_size=self.world_size)
        return workspace.get_received_tensor_payload(id(context.tensor), index, view, self.config, dtype=self.dtype,
                                                     world_size=self.world_size)

    def _send_buffer(self, view: Any, workspace: Any, context: RingSubmissionContext) -> Any:
        buffer = self._payload_buffer("send", context.quant_index, view, workspace, context)
        context.quant_index += 1
        return buffer

    # ---- launches in the active payload format ------------------------------ #
    def _bind_quantize(self, view: Any, payload: Any) -> Any:
        g = self.config.group_size
        if self._wire_direct:
            from lowbit_comm_amd.hip import cuda_wire

            self._whole_groups(view)
            return cuda_wire.bind_quant_pack(view, payload, group_size=g, compact=self.config.compact)
        from lowbit_comm_amd.hip import ops

        return ops.bind_quant_pack_payload(view, payload, group_size=g)

    def _bind_step(self, received: Any, view: Any, send: Any, reduce_op: str, divisor: float) -> Any:
        g = self.config.group_size
        if self._wire_direct:
            from lowbit_comm_amd.hip import cuda_wire

            self._whole_groups(view)
            return cuda_wire.bind_ring_step(received, view, send, group_size=g, compact=self.config.compact,
                                            reduce_op=reduce_op, divisor=divisor)
        from lowbit_comm_amd.hip import ops

        return ops.bind_ring_step(received, view, send, group_size=g, reduce_op=reduce_op, divisor=divisor)

    # ---- steps ------------------------------------------------------------- #
    def quant_pack(self, tensor: Any, chunk: ChunkRange, workspace: Any, *, context: RingSubmissionContext) -> Any:
        from lowbit_comm_amd.hip import ops

        staged, context.staged = context.staged, None
        if staged is not None and staged[0] == (chunk.start, chunk.stop):
            return staged[1]
        if self._facade:
            return self._facade_quantize(tensor, chunk, workspace, context)
        plan, key = context.plan, ("quantize", context.quant_index, chunk.start, chunk.stop)
        bound = None if plan is None else plan.get(key)
        if bound is None:
            view = _view(tensor, chunk)
            payload = self._send_buffer(view, workspace, context)
            bound = (self._bind_quantize(view, payload), payload)
            if plan is not None:
                plan[key] = bound
        else:
            context.quant_index += 1
        if not bound[0](context.raw_stream):
            raise RuntimeError("quantize+pack has no kernel for this configuration")
        if context.program is not None:
            context.program.append(("launch", bound[0]))
        return bound[1]

    def send_recv(self, payload: Any, *, send_peer: int, recv_peer: int, recv_chunk: ChunkRange, workspace: Any,
                  context: RingSubmissionContext) -> tuple[Any, Any]:
        world = self.world_size
        if not (0 <= send_peer < world and 0 <= recv_peer < world):
            raise ValueError("P2P peer must be a valid group-local rank")
        index = context.recv_index
        context.recv_index = index + 1
        received = None if context.plan is None else context.plan.get(("recv", index))
        if received is None:
            # sized for the chunk that arrives, which is shorter than the one sent when it is the ragged last chunk
            received = self._payload_buffer("recv", index, _view(context.tensor, recv_chunk), workspace, context)
        handle = self._exchange(payload, received, send_peer=send_peer, recv_peer=recv_peer, stream=context.stream)
        if context.program is not None:
            context.program.append(("exchange", payload, received, send_peer, recv_peer))
        return received, handle

    def _step(self, tensor: Any, received: Any, chunk: ChunkRange, workspace: Any, context: RingSubmissionContext,
              dependency: Any, *, reduce_op: str, divisor: float, another_hop: bool | None = None) -> Any:
        """``another_hop``: the updated chunk is sent on before anything else changes it, so its payload is worth
        producing in the same launch (default: every hop of a ring but the last)."""
        from lowbit_comm_amd.hip import ops

        dependency.wait_stream(context.stream)
        context.steps_done += 1
        if self._facade:
            return self._facade_step(tensor, received, chunk, context, reduce_op=reduce_op, divisor=divisor)
        if another_hop is None:
            another_hop = context.steps_done < 2 * (self.world_size - 1)
        plan, key = context.plan, ("step", context.steps_done, chunk.start, chunk.stop, received.data_ptr())
        bound = None if plan is None else plan.get(key)
        if bound is None:
            view = _view(tensor, chunk)
            g = self.config.group_size
            if self.fuse_steps:
                send = self._send_buffer(view, workspace, context) if another_hop else None
                launches = (self._bind_step(received, view, send, reduce_op, divisor),)
            else:
                send = None
                launches = (ops.bind_dequant(*ops.split_payload(received, view.numel(), g), view, group_size=g,
                                             reduce_op=reduce_op),)
            bound = (launches, view, send)
            if plan is not None:
                plan[key] = bound
        elif bound[2] is not None:
            context.quant_index += 1
        launches, view, send = bound
        for launch in launches:
            if not launch(context.raw_stream):
                raise RuntimeError("the ring step has no kernel for this configuration")
            if context.program is not None:
                context.program.append(("launch", launch))
        if not self.fuse_steps and divisor != 1.0:
            import torch

            with torch.cuda.stream(context.stream):
                ops.true_divide_(view, divisor)
            if context.program is not None:
                context.program.append(("divide", view, divisor))
        context.staged = ((chunk.start, chunk.stop), send) if send is not None else None
        return view

    # ---- the same steps through the codec facade of a native module -------- #
    def _whole_groups(self, view: Any) -> None:
        from lowbit_comm_amd.exceptions import UnsupportedCollective

        if view.numel() % self.config.group_size != 0:
            raise UnsupportedCollective(
                "topology_all_reduce",
                reason=f"the module's in-place decode needs group-aligned chunks; numel={view.numel()}, "
                       f"group_size={self.config.group_size}")

    def _facade_quantize(self, tensor: Any, chunk: ChunkRange, workspace: Any, context: RingSubmissionContext) -> Any:
        import torch

        from lowbit_comm_amd.quantization.codec import quantize_tensor

        view = _view(tensor, chunk)
        self._whole_groups(view)
        payload = self._send_buffer(view, workspace, context)
        with torch.cuda.stream(context.stream):
            quantize_tensor(view, self.config, extension_status=self.extension_status, output=payload)
        return payload

    def _facade_step(self, tensor: Any, received: Any, chunk: ChunkRange, context: RingSubmissionContext, *,
                     reduce_op: str, divisor: float) -> Any:
        import torch

        from lowbit_comm_amd.quantization.codec import dequantize_tensor

        view = _view(tensor, chunk)
        self._whole_groups(view)
        portable = getattr(getattr(self.extension_status, "module", None), "NATIVE_WIRE_FORMAT", "native") == "portable"
        with torch.cuda.stream(context.stream):
            dequantize_tensor(received, (view.numel(),), self.config, dtype=self.dtype,
                              extension_status=self.extension_status, output=view, reduce_op=reduce_op)
            if divisor != 1.0:
                if portable:
                    from lowbit_comm_amd.hip.ops import true_divide_

                    true_divide_(view, divisor)      # the CPU codec's true division
                else:
                    view.div_(int(divisor))          # what a rank on the CUDA extension computes on its device
        return view

    def fused_reduce(self, tensor: Any, received: Any, chunk: ChunkRange, contributors: tuple[int, ...],
                     workspace: Any, *, context: RingSubmissionContext, dependency: Any) -> Any:
        last = len(contributors) == self.world_size - 1
        out = self._step(tensor, received, chunk, workspace, context, dependency, reduce_op="sum",
                         divisor=float(self.world_size) if last else 1.0)
        if last:
            context.mean_applied = True
        return out

    def apply_broadcast(self, tensor: Any, received: Any, chunk: ChunkRange, workspace: Any, *,
                        context: RingSubmissionContext, dependency: Any) -> Any:
        return self._step(tensor, received, chunk, workspace, context, dependency, reduce_op="none", divisor=1.0)


# --------------------------------------------------------------------------- #
# every rank of a ring on one device
# --------------------------------------------------------------------------- #
class _EventHandle:
    def __init__(self, event: Any) -> None:
        self._event = event

    def query(self) -> bool:
        return bool(self._event.query())

    def is_completed(self) -> bool:
        return self.query()

    def wait(self) -> None:
        self._event.wait()

    def wait_stream(self, stream: Any) -> None:
        stream.wait_event(self._event)


class LoopbackRing:
    """All W ranks of a ring in one process on one device, one host thread per rank: the exchange is a
    device-to-device copy ordered by events, standing in for the links between GPUs (tests, single-GPU
    measurements).  ``exchange_for(rank)`` is the callable a rank's runtime takes; every rank must reach every
    step, as with a real collective.  A rank that fails calls :meth:`abort` so the others do not wait for it."""

    def __init__(self, world_size: int, *, timeout: float = 120.0) -> None:
        self.world_size = world_size
        self._meet = threading.Barrier(world_size, timeout=timeout)
        self._posted: list = [None] * world_size
        self._taken: list = [None] * world_size

    def abort(self) -> None:
        self._meet.abort()

    def exchange_for(self, rank: int) -> Callable[..., Any]:
        import torch

        def exchange(payload: Any, received: Any, *, send_peer: int, recv_peer: int, stream: Any) -> Any:
            ready = torch.cuda.Event()
            ready.record(stream)
            self._posted[rank] = (payload, ready, send_peer)
            self._meet.wait()
            source, source_ready, addressed_to = self._posted[recv_peer]
            if addressed_to != rank:
                self._meet.abort()
                raise RuntimeError(f"rank {recv_peer} sent to {addressed_to}, rank {rank} expected its payload")
            if source.numel() != received.numel():
                self._meet.abort()
                raise RuntimeError("payload sizes of sender and receiver differ")
            stream.wait_event(source_ready)
            with torch.cuda.stream(stream):
                received.copy_(source, non_blocking=True)
            copied = torch.cuda.Event()
            copied.record(stream)
            self._taken[rank] = copied
            self._meet.wait()
            stream.wait_event(self._taken[send_peer])     # the send is over once the receiver has its copy
            return _EventHandle(copied)

        return exchange


def make_pipelined_ring_executor(*, config: CompressionConfig, dtype: str, numel: int, world_size: int, rank: int,
                                 exchange: Callable[..., Any], pool: Any | None = None,
                                 completion_manager: Any | None = None, device: str = "cuda:0",
                                 fuse_steps: bool = True, max_plans: int = 16,
                                 extension_status: Any | None = None, graph_replay: bool = False,
                                 stream: Any | None = None) -> PipelinedRingExecutor:
    """Plan, schedule, runtime, pooled workspaces and executor of one rank for buckets of ``numel`` elements.

    ``stream``: the stream the ring's launches go to.  ``None`` gives the runtime a stream of its own, which lets
    the ring overlap with the caller's compute at the price of an event hand-off in each direction per bucket;
    the caller's own stream (``torch.cuda.current_stream()``) makes a bucket's ring plain stream-ordered work."""
    from lowbit_comm_amd.hip.completion import HipCompletionManager
    from lowbit_comm_amd.hip.workspace import ShardWorkspaceProvider, create_torch_workspace_pool

    manager = completion_manager if completion_manager is not None else HipCompletionManager()
    plan = compile_chunk_plan(original_numel=numel, world_size=world_size)
    schedule = compile_pipelined_ring_schedule(chunk_plan=plan, rank=rank)
    runtime = HipPipelinedRingRuntime(config=config, dtype=dtype, world_size=world_size, rank=rank, exchange=exchange,
                                      completion_manager=manager, fuse_steps=fuse_steps, max_plans=max_plans,
                                      extension_status=extension_status, graph_replay=graph_replay, stream=stream)
    provider = ShardWorkspaceProvider(pool if pool is not None else create_torch_workspace_pool(), backend="hip",
                                      collective="all_reduce", strategy="pipelined_ring", device=device)

    def session_for(tensor: Any) -> Any:
        del tensor
        runtime._ready()
        return provider.begin(stream=runtime.stream)

    return PipelinedRingExecutor(schedule=schedule, runtime=runtime, workspace_session_factory=session_for,
                                 completion_manager=manager)


def make_pipelined_ring_transport(*, world_size: int, rank: int, exchange: Callable[..., Any],
                                  max_executors: int = 16, fuse_steps: bool = True, max_plans: int = 16,
                                  completion_manager: Any | None = None, pool: Any | None = None) -> Callable[..., Any]:
    """The callable ``create_ddp_comm_hook(strategy="topology", topology_all_reduce=...)`` expects, over the ring.

    ``transport(tensor, *, config, op, async_op=False, dtype=None, extension_status=None)`` averages ``tensor`` over
    the ring in place and returns it, ordered on the caller's current stream (``async_op``: the executor's work
    object, whose ``wait()`` returns the tensor).  The ring computes the mean, as the reference's executor does
    (the division sits on the hop that completes the sum, ``ccdl_comm/cuda/transports/torch_topology.py:287-289``);
    any other ``op`` is refused.  One executor is kept per (element count, dtype, device, group size)."""
    from collections import OrderedDict

    from lowbit_comm_amd.exceptions import UnsupportedCollective

    executors: OrderedDict = OrderedDict()

    def transport(tensor: Any, *, config: CompressionConfig, op: str = "mean", async_op: bool = False,
                  dtype: str | None = None, extension_status: Any | None = None) -> Any:
        del extension_status                      # the runtime calls the C ABI directly
        from lowbit_comm_amd.hip import ops

        if op != "mean":
            raise UnsupportedCollective(f"pipelined_ring:{op}", reason="the quantized ring computes the mean")
        name = ops.DTYPE_NAMES.get(tensor.dtype)
        if name is None or (dtype is not None and dtype != name):
            raise ValueError(f"the ring reduces in the bucket's dtype; got dtype={dtype!r} for {tensor.dtype}")
        key = (tensor.numel(), name, str(tensor.device), config.group_size)
        executor = executors.get(key)
        if executor is None:
            executor = executors[key] = make_pipelined_ring_executor(
                config=config, dtype=name, numel=tensor.numel(), world_size=world_size, rank=rank, exchange=exchange,
                pool=pool, completion_manager=completion_manager, device=str(tensor.device), fuse_steps=fuse_steps,
                max_plans=max_plans)
            while len(executors) > max_executors:
                executors.popitem(last=False)
        else:
            executors.move_to_end(key)
        work = executor.run(tensor)
        return work if async_op else work.wait()

    transport.executors = executors
    return transport
