"""Quantized tree all-reduce: compiled schedule, executor and the gfx950 runtime of its compute steps.

Counterparts in the reference: ``TreeEdge``, ``TreeSchedule``, ``compile_tree_schedule`` and ``TreeExecutor``
(``ccdl_comm/cuda/transports/tree.py:19-320``) and ``TorchTreeRuntime``
(``ccdl_comm/cuda/transports/torch_topology.py:319-415``); the reference's compiler takes the tree whenever the
bucket does not split into group-aligned ring chunks (``ccdl_comm/cuda/compiler.py:212-229``).

The ranks form a binary heap relative to the root: logical rank ``k = (rank - root) mod W`` has parent
``(k - 1) // 2``.  Payloads of the whole bucket climb the edges from the highest logical rank down (a parent adds
its children in that order), the root divides by W, and the mean descends the same edges in reverse, quantized
again at every level.  On gfx950 every step that changes the bucket and is followed by a send is one launch of the
ring-step kernel (``lbc_ring_step``: decode, accumulate, the root's division, and the quantize+pack of the result);
a payload produced that way serves every child it goes to, where the reference quantizes once per child.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable

from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.hip.chunk_plan import ChunkPlan, ChunkRange, compile_chunk_plan
from lowbit_comm_amd.hip.ring import (
    HipPipelinedRingRuntime,
    RingSubmissionContext,
    TopologyExecutor,
    _natural,
    _rank_of,
    _Submission,
)


@dataclass(frozen=True)
class TreeEdge:
    """Child -> parent; walked the other way when the mean comes down."""

    child_rank: int
    parent_rank: int

    def __post_init__(self) -> None:
        _natural(self.child_rank, "child_rank")
        _natural(self.parent_rank, "parent_rank")
        if self.child_rank == self.parent_rank:
            raise ValueError("child_rank and parent_rank must differ")


def _heap_edges(world_size: int, root: int) -> tuple[TreeEdge, ...]:
    def rank_of(logical: int) -> int:
        return (root + logical) % world_size

    return tuple(TreeEdge(child_rank=rank_of(k), parent_rank=rank_of((k - 1) // 2)) for k in reversed(range(1, world_size)))


@dataclass(frozen=True)
class TreeSchedule:
    """One rank's view of the tree; only the deterministic topology for (world size, root) is accepted."""

    chunk_plan: ChunkPlan
    rank: int
    root: int
    parent: int | None
    children: tuple[int, ...]
    reduce_edges: tuple[TreeEdge, ...]
    broadcast_edges: tuple[TreeEdge, ...]

    def __post_init__(self) -> None:
        if not isinstance(self.chunk_plan, ChunkPlan):
            raise TypeError("chunk_plan must be a ChunkPlan")
        world = self.chunk_plan.world_size
        _rank_of(self.rank, world, "rank")
        _rank_of(self.root, world, "root")
        edges = _heap_edges(world, self.root)
        if self.reduce_edges != edges:
            raise ValueError("reduce_edges must match the deterministic tree topology")
        if self.broadcast_edges != edges[::-1]:
            raise ValueError("broadcast_edges must reverse the reduce edge order")
        above = [e.parent_rank for e in edges if e.child_rank == self.rank]
        if self.parent != (above[0] if above else None):
            raise ValueError("parent must match the deterministic tree topology")
        if self.children != tuple(e.child_rank for e in edges if e.parent_rank == self.rank):
            raise ValueError("children must match the deterministic tree topology")

    @property
    def local_chunk(self) -> ChunkRange:
        return self.chunk_plan.chunk_for_rank(self.rank)


def compile_tree_schedule(*, chunk_plan: ChunkPlan, rank: int, root: int = 0) -> TreeSchedule:
    if not isinstance(chunk_plan, ChunkPlan):
        raise TypeError("chunk_plan must be a ChunkPlan")
    world = chunk_plan.world_size
    _rank_of(rank, world, "rank")
    _rank_of(root, world, "root")
    edges = _heap_edges(world, root)
    above = [e.parent_rank for e in edges if e.child_rank == rank]
    return TreeSchedule(chunk_plan=chunk_plan, rank=rank, root=root, parent=above[0] if above else None,
                        children=tuple(e.child_rank for e in edges if e.parent_rank == rank), reduce_edges=edges,
                        broadcast_edges=edges[::-1])


def rank_actions(schedule: TreeSchedule) -> tuple[tuple[str, TreeEdge], ...]:
    """What this rank does, in order: ``("reduce", edge)`` receive a child's payload and add it,
    ``("send_up", edge)``, ``("receive_down", edge)`` take the mean from the parent, ``("send_down", edge)``."""
    me = schedule.rank
    climb = [("reduce" if e.parent_rank == me else "send_up", e) for e in schedule.reduce_edges
             if me in (e.parent_rank, e.child_rank)]
    descend = [("receive_down" if e.child_rank == me else "send_down", e) for e in schedule.broadcast_edges
               if me in (e.parent_rank, e.child_rank)]
    return tuple(climb + descend)


class TreeExecutor(TopologyExecutor):
    """Walks the reduce edges, then the broadcast edges, and enqueues this rank's part of each: the runtime
    protocol and call order of ``ccdl_comm/cuda/transports/tree.py:75-281``."""

    schedule_type = TreeSchedule

    def _enqueue(self, submission: _Submission) -> None:
        runtime, tensor, context, workspace = self._runtime, submission.tensor, submission.context, submission.workspace
        for action, edge in rank_actions(self.schedule):
            if action in ("reduce", "receive_down"):
                peer = edge.child_rank if action == "reduce" else edge.parent_rank
                received, handle = runtime.receive(peer=peer, edge=edge, workspace=workspace, context=context)
                submission.keep(received)
                submission.after_p2p(handle)
                apply = runtime.fused_reduce if action == "reduce" else runtime.apply_broadcast
                submission.after(apply(tensor, received, edge, workspace, context=context, dependency=handle))
            else:
                peer = edge.parent_rank if action == "send_up" else edge.child_rank
                payload = runtime.quant_pack(tensor, edge, workspace, context=context)
                submission.keep(payload)
                submission.after_p2p(runtime.send(payload, peer=peer, edge=edge, workspace=workspace, context=context))


class HipTreeRuntime(HipPipelinedRingRuntime):
    """The tree's coarse operations on one gfx950 device.  ``send(payload, peer=, stream=) -> handle`` and
    ``recv(received, peer=, stream=) -> handle`` are the injected point-to-point calls.  Shares buffers, plans, the
    fused step and the facade mode (``extension_status=``) with the ring runtime; the schedule tells it which
    steps are followed by a send, and which step completes the sum at the root."""

    def __init__(self, *, schedule: TreeSchedule, config: CompressionConfig, dtype: str, send: Callable[..., Any],
                 recv: Callable[..., Any], **options: Any) -> None:
        if not isinstance(schedule, TreeSchedule):
            raise TypeError("schedule must be a TreeSchedule")
        for name, fn in (("send", send), ("recv", recv)):
            if not callable(fn):
                raise TypeError(f"{name} must be callable")
        super().__init__(config=config, dtype=dtype, world_size=schedule.chunk_plan.world_size, rank=schedule.rank,
                         exchange=send, **options)
        self.schedule = schedule
        self._send, self._recv = send, recv
        actions = rank_actions(schedule)
        changing = [i for i, (name, _) in enumerate(actions) if name in ("reduce", "receive_down")]
        # per step that changes the bucket (in order): is the very next action a send?
        self._sent_next = tuple(i + 1 < len(actions) and actions[i + 1][0].startswith("send") for i in changing)
        reduces = [k for k, i in enumerate(changing) if actions[i][0] == "reduce"]
        self._completes_sum = reduces[-1] if schedule.parent is None and reduces else None
        self._whole = ChunkRange(0, schedule.chunk_plan.original_numel)

    def create_submission_context(self, tensor: Any) -> RingSubmissionContext:
        context = super().create_submission_context(tensor)
        if tensor.numel() != self._whole.stop:
            raise RuntimeError(f"the schedule was compiled for {self._whole.stop} elements, the tensor has {tensor.numel()}")
        return context

    # ---- sends ------------------------------------------------------------- #
    def quant_pack(self, tensor: Any, edge: TreeEdge, workspace: Any, *, context: RingSubmissionContext) -> Any:
        staged = context.staged                       # stays valid until the next step changes the bucket
        if staged is not None:
            return staged[1]
        if edge.parent_rank == self.rank and not context.mean_applied:
            self._divide(tensor, context)             # only reached when the steps are not fused
        payload = super().quant_pack(tensor, self._whole, workspace, context=context)
        if not self._facade:
            context.staged = ((self._whole.start, self._whole.stop), payload)
        return payload

    def _divide(self, tensor: Any, context: RingSubmissionContext) -> None:
        import torch

        from lowbit_comm_amd.hip.ops import true_divide_

        module = getattr(self.extension_status, "module", None)
        with torch.cuda.stream(context.stream):
            if self.extension_status is None or getattr(module, "NATIVE_WIRE_FORMAT", "native") == "portable":
                true_divide_(tensor.reshape(-1), float(self.world_size))
            else:
                tensor.div_(self.world_size)          # what a rank on the CUDA extension computes on its device
        context.mean_applied = True
        context.staged = None

    def send(self, payload: Any, *, peer: int, edge: TreeEdge, workspace: Any, context: RingSubmissionContext) -> Any:
        del edge, workspace
        _rank_of(peer, self.world_size, "P2P peer")
        return self._send(payload, peer=peer, stream=context.stream)

    # ---- receives ---------------------------------------------------------- #
    def receive(self, *, peer: int, edge: TreeEdge, workspace: Any, context: RingSubmissionContext) -> tuple[Any, Any]:
        del edge
        _rank_of(peer, self.world_size, "P2P peer")
        index = context.recv_index
        context.recv_index = index + 1
        received = None if context.plan is None else context.plan.get(("recv", index))
        if received is None:
            received = self._payload_buffer("recv", index, context.tensor.reshape(-1), workspace, context)
        return received, self._recv(received, peer=peer, stream=context.stream)

    def _change(self, tensor: Any, received: Any, workspace: Any, context: RingSubmissionContext, dependency: Any,
                reduce_op: str) -> Any:
        step = context.steps_done                     # index among the steps that change the bucket
        completes = step == self._completes_sum
        fused_division = completes and self.fuse_steps
        out = self._step(tensor, received, self._whole, workspace, context, dependency, reduce_op=reduce_op,
                         divisor=float(self.world_size) if fused_division else 1.0,
                         another_hop=self._sent_next[step])
        if fused_division or reduce_op == "none":
            context.mean_applied = True
        return out

    def fused_reduce(self, tensor: Any, received: Any, edge: TreeEdge, workspace: Any, *,
                     context: RingSubmissionContext, dependency: Any) -> Any:
        del edge
        return self._change(tensor, received, workspace, context, dependency, "sum")

    def apply_broadcast(self, tensor: Any, received: Any, edge: TreeEdge, workspace: Any, *,
                        context: RingSubmissionContext, dependency: Any) -> Any:
        del edge
        return self._change(tensor, received, workspace, context, dependency, "none")


def make_tree_executor(*, config: CompressionConfig, dtype: str, numel: int, world_size: int, rank: int,
                       send: Callable[..., Any], recv: Callable[..., Any], root: int = 0, pool: Any | None = None,
                       completion_manager: Any | None = None, device: str = "cuda:0", fuse_steps: bool = True,
                       max_plans: int = 16, extension_status: Any | None = None) -> TreeExecutor:
    """Plan, schedule, runtime, pooled workspaces and executor of one rank for buckets of ``numel`` elements."""
    from lowbit_comm_amd.hip.completion import HipCompletionManager
    from lowbit_comm_amd.hip.workspace import ShardWorkspaceProvider, create_torch_workspace_pool

    manager = completion_manager if completion_manager is not None else HipCompletionManager()
    schedule = compile_tree_schedule(chunk_plan=compile_chunk_plan(original_numel=numel, world_size=world_size),
                                     rank=rank, root=root)
    runtime = HipTreeRuntime(schedule=schedule, config=config, dtype=dtype, send=send, recv=recv,
                             completion_manager=manager, fuse_steps=fuse_steps, max_plans=max_plans,
                             extension_status=extension_status)
    provider = ShardWorkspaceProvider(pool if pool is not None else create_torch_workspace_pool(), backend="hip",
                                      collective="all_reduce", strategy="topology_tree", device=device)

    def session_for(tensor: Any) -> Any:
        del tensor
        runtime._ready()
        return provider.begin(stream=runtime.stream)

    return TreeExecutor(schedule=schedule, runtime=runtime, workspace_session_factory=session_for,
                        completion_manager=manager)


class LoopbackMesh:
    """Point-to-point links between W ranks that live in one process on one device (a host thread per rank), for
    tests and single-GPU measurements: ``send_for(rank)`` / ``recv_for(rank)`` are the callables a rank's runtime
    takes.  A send stages a copy of the payload and posts it with an event; the matching receive waits for that
    event on its own stream and copies the bytes into its buffer.  Messages between a pair of ranks arrive in the
    order they were sent."""

    def __init__(self, world_size: int, *, timeout: float = 120.0) -> None:
        import queue

        self.world_size = world_size
        self.timeout = timeout
        self._links = {(a, b): queue.Queue() for a in range(world_size) for b in range(world_size) if a != b}

    def send_for(self, rank: int) -> Callable[..., Any]:
        import torch

        from lowbit_comm_amd.hip.ring import _EventHandle

        def send(payload: Any, *, peer: int, stream: Any) -> Any:
            with torch.cuda.stream(stream):
                staged = payload.clone()
            posted = torch.cuda.Event()
            posted.record(stream)
            self._links[(rank, peer)].put((staged, posted))
            return _EventHandle(posted)

        return send

    def recv_for(self, rank: int) -> Callable[..., Any]:
        import torch

        from lowbit_comm_amd.hip.ring import _EventHandle

        def recv(received: Any, *, peer: int, stream: Any) -> Any:
            staged, posted = self._links[(peer, rank)].get(timeout=self.timeout)
            if staged.numel() != received.numel():
                raise RuntimeError("payload sizes of sender and receiver differ")
            stream.wait_event(posted)
            with torch.cuda.stream(stream):
                received.copy_(staged, non_blocking=True)
            staged.record_stream(stream)
            arrived = torch.cuda.Event()
            arrived.record(stream)
            return _EventHandle(arrived)

        return recv


class _BothHandles:
    """The send and the receive of one ring hop as one dependency."""

    def __init__(self, *handles: Any) -> None:
        self._handles = handles

    def query(self) -> bool:
        return all(bool(h.query()) for h in self._handles)

    def is_completed(self) -> bool:
        return self.query()

    def wait_stream(self, stream: Any) -> None:
        for handle in self._handles:
            handle.wait_stream(stream)


def make_topology_transport(*, world_size: int, rank: int, send: Callable[..., Any], recv: Callable[..., Any],
                            root: int = 0, max_executors: int = 16, fuse_steps: bool = True, max_plans: int = 16,
                            completion_manager: Any | None = None, pool: Any | None = None,
                            extension_status: Any | None = None) -> Callable[..., Any]:
    """The callable ``create_ddp_comm_hook(strategy="topology", topology_all_reduce=...)`` expects, over the ring or
    the tree as the reference's compiler chooses between them (``ccdl_comm/cuda/compiler.py:212-229``): the ring
    when the bucket splits into W chunks of whole groups, the tree otherwise - every rank of a job, whatever it
    runs on, must make the same choice.  ``send(payload, peer=, stream=)`` / ``recv(received, peer=, stream=)`` are
    the point-to-point calls (a ring hop posts one of each).  Averages ``tensor`` in place and returns it
    (``async_op``: the executor's work object); any ``op`` but ``"mean"`` is refused."""
    from collections import OrderedDict

    from lowbit_comm_amd.exceptions import UnsupportedCollective
    from lowbit_comm_amd.hip.ring import make_pipelined_ring_executor

    executors: OrderedDict = OrderedDict()

    def ring_exchange(payload: Any, received: Any, *, send_peer: int, recv_peer: int, stream: Any) -> Any:
        return _BothHandles(send(payload, peer=send_peer, stream=stream), recv(received, peer=recv_peer, stream=stream))

    def transport(tensor: Any, *, config: CompressionConfig, op: str = "mean", async_op: bool = False,
                  dtype: str | None = None, **hook_arguments: Any) -> Any:
        del hook_arguments                        # the hook also hands over its own extension_status=
        from lowbit_comm_amd.hip import ops

        if op != "mean":
            raise UnsupportedCollective(f"topology_all_reduce:{op}", reason="the quantized ring and tree compute the mean")
        name = ops.DTYPE_NAMES.get(tensor.dtype)
        if name is None or (dtype is not None and dtype != name):
            raise ValueError(f"the topology schedules reduce in the bucket's dtype; got dtype={dtype!r} for {tensor.dtype}")
        n = tensor.numel()
        key = (n, name, str(tensor.device), config.group_size)
        executor = executors.get(key)
        if executor is None:
            aligned = world_size >= 2 and n % world_size == 0 and (n // world_size) % config.group_size == 0
            common = dict(config=config, dtype=name, numel=n, world_size=world_size, rank=rank, pool=pool,
                          completion_manager=completion_manager, device=str(tensor.device), fuse_steps=fuse_steps,
                          max_plans=max_plans, extension_status=extension_status)
            executor = (make_pipelined_ring_executor(exchange=ring_exchange, **common) if aligned
                        else make_tree_executor(send=send, recv=recv, root=root, **common))
            executors[key] = executor
            while len(executors) > max_executors:
                executors.popitem(last=False)
        else:
            executors.move_to_end(key)
        work = executor.run(tensor)
        return work if async_op else work.wait()

    transport.executors = executors
    return transport
