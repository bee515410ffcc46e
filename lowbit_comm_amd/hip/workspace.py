"""Stream-safe pool of reusable device workspaces for the compression path.

Behaviour follows the reference's ``CudaWorkspacePool`` family (``ccdl_comm/cuda/workspace.py:18-627``):

* a buffer is identified by a :class:`WorkspaceKey` (collective, strategy, shape, dtype, world size,
  codec policy, chunk, kind, device); ``acquire`` reuses an idle buffer of the same key (oldest first),
  else takes over a buffer of that key whose previous user has *released it with a completion that is
  still pending* by making the acquiring stream wait on that completion (no host sync), else allocates;
* ``release`` hands the buffer back together with a completion object (``query() -> bool``, optional
  ``wait_stream(stream)``); it only becomes idle once ``query()`` is true, checked lazily on later calls;
* idle buffers are evicted least-recently-idled first when entry or byte budgets are exceeded;
  in-flight buffers never are;
* every use calls ``record_stream`` on the buffer so the caching allocator cannot recycle it early.

Completions for HIP streams come from :class:`StreamOrderedCompletion` (nothing recorded while the buffer stays on
one stream) or :class:`EventCompletion` (a ``torch.cuda.Event`` recorded on the
releasing stream).  The pool itself is host-side bookkeeping and works with any objects that provide
the small protocols above, which is how the CPU tests drive it.
"""
from __future__ import annotations

from collections import OrderedDict, deque
from collections.abc import Callable
from dataclasses import dataclass
from math import prod
from threading import Lock
from typing import Any

from lowbit_comm_amd.config import CompressionConfig
from lowbit_comm_amd.quantization.sizing import estimate_quantized_size

_ELEMENT_BYTES = {"float64": 8, "double": 8, "int64": 8, "float32": 4, "float": 4, "fp32": 4, "int32": 4,
                  "float16": 2, "half": 2, "fp16": 2, "bfloat16": 2, "bf16": 2, "int16": 2}


def _element_bytes(dtype: str) -> int:
    return _ELEMENT_BYTES.get(dtype.lower().removeprefix("torch."), 1)


@dataclass(frozen=True)
class WorkspaceKey:
    """Everything that can change the size or the meaning of a workspace allocation."""

    backend: str
    collective: str
    strategy: str
    shape_class: tuple[int, ...]
    dtype: str
    world_size: int
    bit: int
    group_size: int
    chunk_config: tuple[int, ...]
    workspace_kind: str
    device: str = "cuda"

    def __post_init__(self) -> None:
        for name in ("backend", "collective", "strategy", "workspace_kind"):
            if not getattr(self, name):
                raise ValueError(f"{name} must not be empty")
        if any(dim < 0 for dim in self.shape_class):
            raise ValueError("shape_class dimensions must be >= 0")
        for name in ("world_size", "bit", "group_size"):
            if getattr(self, name) < 1:
                raise ValueError(f"{name} must be >= 1")

    @property
    def estimated_bytes(self) -> int:
        """Size to account for when the allocated object cannot report its own."""
        return prod(self.shape_class) * _element_bytes(self.dtype)


@dataclass(frozen=True)
class WorkspaceStats:
    hits: int
    misses: int
    evictions: int
    cached_bytes: int
    in_flight_bytes: int


class _Slot:
    __slots__ = ("ident", "key", "buffer", "size_bytes", "completion", "sweeps")

    def __init__(self, ident: int, key: WorkspaceKey, buffer: Any, size_bytes: int) -> None:
        self.ident = ident
        self.key = key
        self.buffer = buffer
        self.size_bytes = size_bytes
        self.completion: Any | None = None
        self.sweeps = 0          # polls that found the completion pending since the release


def _nbytes(buffer: Any, fallback: int) -> int:
    nbytes = getattr(buffer, "nbytes", None)
    if nbytes is not None:
        return int(nbytes)
    numel, size = getattr(buffer, "numel", None), getattr(buffer, "element_size", None)
    if callable(numel) and callable(size):
        return int(numel()) * int(size())
    return fallback


# A completion that offers peek() may never turn true by itself: a StreamOrderedCompletion records its event only when
# somebody asks with query().  A released buffer that no acquire has taken over after this many polls is therefore
# settled by the pool itself, with query(): the event is recorded once, late, and the following peeks see it.  The
# usual case - the next bucket acquires the same key on the same stream within a few acquires - never gets here and
# pays for no event.
_SETTLE_AFTER_SWEEPS = 8


def _is_done(completion: Any, *, settle: bool = False) -> bool:
    """Has the work behind ``completion`` finished?  A completion may offer ``peek()``, a form of ``query()`` that
    costs the device nothing (see :class:`StreamOrderedCompletion`); the pool's own polling uses it when it is there,
    unless ``settle`` asks for the real answer."""
    peek = getattr(completion, "peek", None)
    if callable(peek) and not settle:
        return bool(peek())
    query = getattr(completion, "query", None)
    return callable(query) and bool(query())


class WorkspaceLease:
    """Exclusive use of one pooled buffer until :meth:`release`."""

    def __init__(self, pool: "HipWorkspacePool", slot: _Slot) -> None:
        self._pool = pool
        self._slot = slot
        self._released = False
        self._lock = Lock()

    @property
    def buffer(self) -> Any:
        return self._slot.buffer

    @property
    def key(self) -> WorkspaceKey:
        return self._slot.key

    @property
    def size_bytes(self) -> int:
        return self._slot.size_bytes

    @property
    def released(self) -> bool:
        with self._lock:
            return self._released

    def release(self, *, completion: Any) -> None:
        """Give the buffer back; it is reusable once ``completion.query()`` is true."""
        with self._lock:
            if self._released:
                raise RuntimeError("workspace lease is already released")
            self._released = True
            try:
                self._pool._give_back(self._slot, completion)
            except BaseException:
                self._released = False
                raise


class HipWorkspacePool:
    """LRU pool whose buffers change hands on stream completions instead of host synchronisation."""

    def __init__(self, *, allocator: Callable[[WorkspaceKey, Any], Any], max_cached_bytes: int | None = None,
                 max_entries: int | None = None) -> None:
        if not callable(allocator):
            raise TypeError("allocator must be callable")
        if max_cached_bytes is not None and max_cached_bytes < 0:
            raise ValueError("max_cached_bytes must be >= 0 or None")
        if max_entries is not None and max_entries < 1:
            raise ValueError("max_entries must be >= 1 or None")
        self._allocator = allocator
        self._max_cached_bytes = max_cached_bytes
        self._max_entries = max_entries
        self._idle: OrderedDict[int, _Slot] = OrderedDict()          # least recently idled first
        self._idle_of_key: dict[WorkspaceKey, deque[int]] = {}
        self._busy: dict[int, _Slot] = {}                            # leased, or released but not yet complete
        self._pending_of_key: dict[WorkspaceKey, deque[int]] = {}    # released with a pending completion
        self._counter = 0
        self._hits = self._misses = self._evictions = 0
        self._cached_bytes = self._busy_bytes = 0
        self._lock = Lock()

    # ---- public ----------------------------------------------------------------------------------
    def acquire(self, key: WorkspaceKey, stream: Any) -> WorkspaceLease:
        if not isinstance(key, WorkspaceKey):
            raise TypeError("key must be a WorkspaceKey")
        with self._lock:
            self._collect_finished()
            slot = self._pop_idle(key)
            if slot is not None:
                self._enter_busy(slot)
                self._hits += 1
            else:
                slot = self._adopt_pending(key, stream)
                if slot is not None:
                    self._hits += 1
                else:
                    buffer = self._allocator(key, stream)
                    slot = _Slot(self._counter, key, buffer, _nbytes(buffer, key.estimated_bytes))
                    self._counter += 1
                    self._misses += 1
                    self._enter_busy(slot)
            record = getattr(slot.buffer, "record_stream", None)
            if callable(record) and stream is not None:
                record(stream)
            return WorkspaceLease(self, slot)

    @property
    def stats(self) -> WorkspaceStats:
        with self._lock:
            self._collect_finished()
            return WorkspaceStats(hits=self._hits, misses=self._misses, evictions=self._evictions,
                                  cached_bytes=self._cached_bytes, in_flight_bytes=self._busy_bytes)

    def clear(self) -> None:
        """Forget idle buffers; buffers still owned by leases or pending work are kept."""
        with self._lock:
            self._idle.clear()
            self._idle_of_key.clear()
            self._cached_bytes = 0

    # ---- internals (lock held) ------------------------------------------------------------------
    def _enter_busy(self, slot: _Slot) -> None:
        self._busy[slot.ident] = slot
        self._busy_bytes += slot.size_bytes

    def _give_back(self, slot: _Slot, completion: Any) -> None:
        if not callable(getattr(completion, "query", None)):
            raise TypeError("completion must provide query()")
        with self._lock:
            if slot.ident not in self._busy:
                raise RuntimeError("workspace lease is not owned by this pool")
            slot.completion = completion
            slot.sweeps = 0
            if _is_done(completion):
                self._become_idle(slot)
            else:
                self._pending_of_key.setdefault(slot.key, deque()).append(slot.ident)

    def _collect_finished(self) -> None:
        for pending in list(self._pending_of_key.values()):
            for ident in list(pending):
                slot = self._busy.get(ident)
                if slot is None or slot.completion is None:
                    continue
                slot.sweeps += 1
                if _is_done(slot.completion, settle=slot.sweeps == _SETTLE_AFTER_SWEEPS):
                    self._become_idle(slot)

    def _forget_pending(self, slot: _Slot) -> None:
        pending = self._pending_of_key.get(slot.key)
        if pending is None:
            return
        try:
            pending.remove(slot.ident)
        except ValueError:
            pass
        if not pending:
            del self._pending_of_key[slot.key]

    def _become_idle(self, slot: _Slot) -> None:
        if self._busy.pop(slot.ident, None) is None:
            return
        self._forget_pending(slot)
        self._busy_bytes -= slot.size_bytes
        slot.completion = None
        self._idle[slot.ident] = slot
        self._idle_of_key.setdefault(slot.key, deque()).append(slot.ident)
        self._cached_bytes += slot.size_bytes
        self._evict()

    def _pop_idle(self, key: WorkspaceKey) -> _Slot | None:
        queue = self._idle_of_key.get(key)
        while queue:
            slot = self._idle.pop(queue.popleft(), None)
            if slot is not None:
                if not queue:
                    del self._idle_of_key[key]
                self._cached_bytes -= slot.size_bytes
                return slot
        self._idle_of_key.pop(key, None)
        return None

    def _adopt_pending(self, key: WorkspaceKey, stream: Any) -> _Slot | None:
        """Take over a released-but-unfinished buffer of ``key`` by ordering ``stream`` after its completion."""
        for ident in list(self._pending_of_key.get(key, ())):
            slot = self._busy.get(ident)
            if slot is None or slot.completion is None:
                continue
            wait_stream = getattr(slot.completion, "wait_stream", None)
            if not callable(wait_stream):
                continue
            wait_stream(stream)
            slot.completion = None
            self._forget_pending(slot)
            return slot          # stays in _busy: ownership moved, bytes already counted
        return None

    def _evict(self) -> None:
        while self._idle and (
                (self._max_entries is not None and len(self._idle) > self._max_entries)
                or (self._max_cached_bytes is not None and self._cached_bytes > self._max_cached_bytes)):
            ident, slot = self._idle.popitem(last=False)
            self._cached_bytes -= slot.size_bytes
            self._evictions += 1
            queue = self._idle_of_key.get(slot.key)
            if queue is not None:
                try:
                    queue.remove(ident)
                except ValueError:
                    pass
                if not queue:
                    del self._idle_of_key[slot.key]


# The reference's class name, for call sites that construct the pool directly.
CudaWorkspacePool = HipWorkspacePool


# --------------------------------------------------------------------------- #
# completions
# --------------------------------------------------------------------------- #
class NoopCompletion:
    """Completion of work that needs no device ordering (host tensors, no GPU)."""

    def query(self) -> bool:
        return True

    def wait(self) -> None:
        return None

    def wait_stream(self, stream: Any) -> None:
        del stream

    def synchronize(self) -> None:
        return None


class EventCompletion:
    """Completion of everything enqueued on ``stream`` so far, as a recorded device event."""

    def __init__(self, stream: Any = None) -> None:
        import torch

        self._event = torch.cuda.Event()
        self._event.record(stream if stream is not None else torch.cuda.current_stream())

    def query(self) -> bool:
        return bool(self._event.query())

    def wait(self) -> None:
        """Order torch's current stream after the event (device-side wait; the host does not block)."""
        self._event.wait()

    def wait_stream(self, stream: Any) -> None:
        """Order ``stream`` after the event (device-side wait; the host does not block)."""
        stream.wait_event(self._event)

    def synchronize(self) -> None:
        self._event.synchronize()


class StreamOrderedCompletion:
    """Completion of everything enqueued on ``stream`` so far, for buffers whose next user is usually that same
    stream.

    No event is recorded when the object is made.  A later acquire on the same stream needs nothing (the stream's
    own order covers it: ``wait_stream`` is a no-op, and the pool hands the buffer over while it is still
    "pending"); only a waiter on another stream, ``query()`` or ``synchronize()`` records the event, at that
    moment - an event recorded later on the stream completes no earlier, so the answer stays correct, merely
    conservative.  ``peek()`` never records.  The reason: on this part a device event between two kernels of one
    stream costs 2.6-2.8 us of GPU time (measured on a stream of 30 us launches with one release per bucket:
    31.3 us per bucket with an event, 28.4 us without)."""

    def __init__(self, stream: Any = None) -> None:
        import torch

        self._stream = stream if stream is not None else torch.cuda.current_stream()
        self._event = None

    def covers(self, stream: Any) -> bool:
        """Is work enqueued on ``stream`` from now on ordered after this completion without any wait?"""
        return stream is not None and stream == self._stream

    def _recorded(self):
        if self._event is None:
            import torch

            self._event = torch.cuda.Event()
            self._event.record(self._stream)
        return self._event

    def peek(self) -> bool:
        return self._event is not None and bool(self._event.query())

    def query(self) -> bool:
        return bool(self._recorded().query())

    def wait(self) -> None:
        import torch

        self.wait_stream(torch.cuda.current_stream())

    def wait_stream(self, stream: Any) -> None:
        if not self.covers(stream):
            stream.wait_event(self._recorded())

    def synchronize(self) -> None:
        self._recorded().synchronize()


class EventCompletionManager:
    """``record_for(value, stream=None)`` -> a completion (the protocol output leases and the asynchronous bucket
    pipeline consume): an :class:`EventCompletion` for GPU values, a :class:`NoopCompletion` otherwise."""

    def record_for(self, value: Any, *, stream: Any = None) -> Any:
        if stream is None and getattr(value, "is_cuda", None) is False:
            return NoopCompletion()          # a host tensor: nothing on the device to order after
        import torch

        if not torch.cuda.is_available():
            return NoopCompletion()
        return EventCompletion(stream)


# --------------------------------------------------------------------------- #
# output lease
# --------------------------------------------------------------------------- #
class HipOutputLease:
    """Ownership of one pooled reduced-shard output: ACQUIRED -> SUBMITTING -> BOUND -> RELEASED.

    The executor that owns the lease (identified by ``owner_token``) marks it used for exactly one run,
    binds the work whose completion authorises release, and releases it after that work completed.
    """

    _ACQUIRED, _SUBMITTING, _BOUND, _RELEASED = "ACQUIRED", "SUBMITTING", "BOUND", "RELEASED"

    def __init__(self, lease: WorkspaceLease, *, owner_token: object, completion_manager: Any,
                 acquisition_stream: Any) -> None:
        if not isinstance(lease, WorkspaceLease):
            raise TypeError("lease must be a WorkspaceLease")
        if owner_token is None:
            raise TypeError("owner_token must not be None")
        if completion_manager is None:
            raise TypeError("completion_manager must not be None")
        self._lease = lease
        self._owner = owner_token
        self._manager = completion_manager
        self._stream = acquisition_stream
        self._state = self._ACQUIRED
        self._work: Any | None = None
        self._lock = Lock()

    @property
    def buffer(self) -> Any:
        return self._lease.buffer

    def _check(self, owner_token: object | None = None, *, check_owner: bool = True) -> None:
        if self._state == self._RELEASED:
            raise RuntimeError("CUDA output lease is already released")
        if check_owner and owner_token is not self._owner:
            raise RuntimeError("CUDA output lease belongs to a different executor")

    def mark_used(self, owner_token: object) -> Any:
        with self._lock:
            self._check(owner_token)
            if self._state != self._ACQUIRED:
                raise RuntimeError("CUDA output lease is already in use")
            self._state = self._SUBMITTING
            return self._lease.buffer

    def bind_work(self, owner_token: object, work: Any) -> None:
        with self._lock:
            self._check(owner_token)
            if self._state != self._SUBMITTING:
                raise RuntimeError("CUDA output lease must be submitting before binding work")
            self._work = work
            self._state = self._BOUND

    def abort_use(self, owner_token: object) -> None:
        with self._lock:
            self._check(owner_token)
            if self._state != self._SUBMITTING:
                raise RuntimeError("CUDA output lease can abort only while submitting")
            self._state = self._ACQUIRED

    def release_after(self, value_or_completion: Any) -> None:
        """Return the storage after the bound work has completed; accepts a completion or a tensor to fence on."""
        with self._lock:
            self._check(check_owner=False)
            if self._state == self._ACQUIRED:
                raise RuntimeError("CUDA output lease must be marked used before release_after")
            if self._state == self._SUBMITTING or self._work is None:
                raise RuntimeError("CUDA output lease must be bound to work before release_after")
            if not _work_done(self._work):
                raise RuntimeError("CUDA output lease cannot release until associated work completes")
            completion = value_or_completion
            if not callable(getattr(completion, "query", None)):
                completion = _record(self._manager, value_or_completion)
            self._finish(completion)

    def release_unused(self) -> None:
        """Return untouched storage, ordered after the stream it was acquired on."""
        with self._lock:
            self._check(check_owner=False)
            if self._state != self._ACQUIRED:
                raise RuntimeError("CUDA output lease cannot release_unused after mark_used")
            self._finish(_record(self._manager, self._lease.buffer, stream=self._stream))

    def _finish(self, completion: Any) -> None:
        before = self._state
        self._state = self._RELEASED
        try:
            self._lease.release(completion=completion)
            self._work = None
        except BaseException:
            self._state = before
            raise


CudaOutputLease = HipOutputLease


def _work_done(work: Any) -> bool:
    for name in ("query", "is_completed"):
        probe = getattr(work, name, None)
        if callable(probe):
            return bool(probe())
    return False


def _record(manager: Any, value: Any, *, stream: Any = None) -> Any:
    record_for = getattr(manager, "record_for", None)
    if not callable(record_for):
        raise TypeError("completion_manager must provide record_for()")
    completion = record_for(value) if stream is None else record_for(value, stream=stream)
    if not callable(getattr(completion, "query", None)):
        raise TypeError("completion_manager.record_for() must return completion with query()")
    return completion


# --------------------------------------------------------------------------- #
# shard sessions: send / recv / reduced workspaces of one shard collective call
# --------------------------------------------------------------------------- #
class ShardWorkspaceProvider:
    """Binds shard-workspace keys (collective, strategy, device) to one executor-owned pool."""

    def __init__(self, pool: HipWorkspacePool, *, backend: str, collective: str, strategy: str, device: str,
                 pool_reduced_output: bool = True) -> None:
        if not isinstance(pool, HipWorkspacePool):
            raise TypeError("pool must be a CudaWorkspacePool")
        self.pool = pool
        self._backend = backend
        self._collective = collective
        self._strategy = strategy
        self._device = device
        self.pool_reduced_output = bool(pool_reduced_output)

    def begin(self, *, stream: Any) -> "ShardWorkspaceSession":
        return ShardWorkspaceSession(self, stream=stream)


class ShardWorkspaceSession:
    """Leases taken during one call; ``release`` returns all of them with one completion."""

    def __init__(self, provider: ShardWorkspaceProvider, *, stream: Any) -> None:
        self._provider = provider
        self._stream = stream
        self._leases: list[WorkspaceLease] = []

    @property
    def leases(self) -> tuple[WorkspaceLease, ...]:
        return tuple(self._leases)

    def _take(self, *, shape: tuple[int, ...], dtype: str, world_size: int, config: CompressionConfig,
              chunk_config: tuple[int, ...], kind: str) -> Any:
        p = self._provider
        key = WorkspaceKey(backend=p._backend, collective=p._collective, strategy=p._strategy, shape_class=shape,
                           dtype=dtype, world_size=world_size, bit=config.bit, group_size=config.group_size,
                           chunk_config=chunk_config, workspace_kind=kind, device=p._device)
        lease = p.pool.acquire(key, self._stream)
        self._leases.append(lease)
        return lease.buffer

    def acquire(self, key: WorkspaceKey) -> Any:
        """Lease a buffer for an explicit key on this session's stream; released with the others."""
        lease = self._provider.pool.acquire(key, self._stream)
        self._leases.append(lease)
        return lease.buffer

    def _payload_bytes(self, tensor: Any, config: CompressionConfig, dtype: str) -> int:
        return estimate_quantized_size(int(tensor.numel()), dtype=dtype, config=config,
                                       wire_format="portable").quantized_bytes

    def get_quantized_chunk(self, bucket_key: Any, chunk_index: int, tensor: Any, config: CompressionConfig, *,
                            dtype: str, world_size: int) -> Any:
        del bucket_key
        return self._take(shape=(self._payload_bytes(tensor, config, dtype),), dtype="uint8", world_size=world_size,
                          config=config, chunk_config=(chunk_index, int(tensor.numel())), kind="send")

    def get_received_payload(self, bucket_key: Any, payload_template: Any, index: int, *, world_size: int,
                             config: CompressionConfig) -> Any:
        del bucket_key
        return self._take(shape=tuple(payload_template.shape), dtype=str(payload_template.dtype),
                          world_size=world_size, config=config, chunk_config=(index,), kind="recv")

    def get_received_tensor_payload(self, bucket_key: Any, index: int, tensor: Any, config: CompressionConfig, *,
                                    dtype: str, world_size: int) -> Any:
        del bucket_key
        return self._take(shape=(self._payload_bytes(tensor, config, dtype),), dtype="uint8", world_size=world_size,
                          config=config, chunk_config=(index, int(tensor.numel())), kind="recv")

    def get_reduced_shard(self, bucket_key: Any, tensor: Any, shape: tuple[int, ...], config: CompressionConfig, *,
                          dtype: str, world_size: int, rank: int) -> Any:
        del bucket_key, dtype
        if not self._provider.pool_reduced_output:
            return None
        numel = prod(shape)
        padded = -(-numel // config.group_size) * config.group_size if numel else 0
        return self._take(shape=(padded,), dtype=str(tensor.dtype), world_size=world_size, config=config,
                          chunk_config=(rank,), kind="reduced")

    def release(self, *, completion: Any) -> None:
        while self._leases:
            self._leases.pop(0).release(completion=completion)


CudaShardWorkspaceProvider = ShardWorkspaceProvider
CudaShardWorkspaceSession = ShardWorkspaceSession


def _allocate_torch(key: WorkspaceKey, stream: Any) -> Any:
    del stream
    import torch

    name = key.dtype.lower().removeprefix("torch.")
    table = {"fp16": torch.float16, "half": torch.float16, "float16": torch.float16, "bf16": torch.bfloat16,
             "bfloat16": torch.bfloat16, "fp32": torch.float32, "float": torch.float32, "float32": torch.float32,
             "uint8": torch.uint8, "int8": torch.int8}
    if name not in table:
        raise ValueError(f"unsupported workspace dtype: {key.dtype!r}")
    return torch.empty(key.shape_class, dtype=table[name], device=key.device)


def create_torch_workspace_pool(*, max_cached_bytes: int | None = None,
                                max_entries: int | None = None) -> HipWorkspacePool:
    """A pool whose misses allocate torch tensors on ``key.device``."""
    return HipWorkspacePool(allocator=_allocate_torch, max_cached_bytes=max_cached_bytes, max_entries=max_entries)
