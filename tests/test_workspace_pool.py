"""Host-side behaviour of the stream-safe workspace pool, driven with fake buffers and completions
(the behaviours the reference pins in tests/cuda/test_cuda_workspace_pool.py:89-590)."""
import threading
from dataclasses import replace

import pytest

from lowbit_comm_amd import CompressionConfig
from lowbit_comm_amd.hip import (
    CudaOutputLease,
    CudaWorkspacePool,
    HipOutputLease,
    HipWorkspacePool,
    ShardWorkspaceProvider,
    WorkspaceKey,
    WorkspaceLease,
    WorkspaceStats,
)

KEY = WorkspaceKey(backend="hip", collective="reduce_scatter", strategy="compressed", shape_class=(1024,),
                   dtype="float16", world_size=4, bit=8, group_size=32, chunk_config=(256, 4), workspace_kind="send")


class Buffer:
    def __init__(self, key):
        self.key = key
        self.nbytes = key.estimated_bytes
        self.recorded_streams = []

    def record_stream(self, stream):
        self.recorded_streams.append(stream)


class Completion:
    def __init__(self, ready=False):
        self.ready = ready
        self.waited = []

    def query(self):
        return self.ready

    def wait_stream(self, stream):
        self.waited.append(stream)


class QueryOnly:
    def __init__(self, ready=False):
        self.ready = ready

    def query(self):
        return self.ready


def make_pool(**kw):
    made = []

    def allocator(key, stream):
        made.append((key, stream))
        return Buffer(key)

    return HipWorkspacePool(allocator=allocator, **kw), made


def test_names_and_key_dimensions():
    assert CudaWorkspacePool is HipWorkspacePool and CudaOutputLease is HipOutputLease
    assert WorkspaceLease.__name__ == "WorkspaceLease" and WorkspaceStats.__name__ == "WorkspaceStats"
    assert KEY.estimated_bytes == 2048
    for change in (dict(backend="cpu"), dict(collective="all_reduce"), dict(strategy="all_gather"),
                   dict(shape_class=(2048,)), dict(dtype="float32"), dict(world_size=2), dict(bit=4),
                   dict(group_size=64), dict(chunk_config=(512, 2)), dict(workspace_kind="recv"), dict(device="cuda:1")):
        assert replace(KEY, **change) != KEY
    for bad in (dict(backend=""), dict(shape_class=(-1,)), dict(world_size=0), dict(bit=0), dict(group_size=0),
                dict(workspace_kind="")):
        with pytest.raises(ValueError):
            replace(KEY, **bad)
    with pytest.raises(TypeError):
        HipWorkspacePool(allocator=None)
    with pytest.raises(ValueError):
        make_pool(max_entries=0)
    with pytest.raises(TypeError, match="WorkspaceKey"):
        make_pool()[0].acquire("key", "s")


def test_completed_workspace_is_reused_and_steady_state_allocates_nothing():
    pool, made = make_pool()
    for _ in range(5):
        lease = pool.acquire(KEY, "s0")
        lease.release(completion=Completion(ready=True))
    stats = pool.stats
    assert len(made) == 1 and (stats.hits, stats.misses) == (4, 1)
    assert stats.cached_bytes == 2048 and stats.in_flight_bytes == 0


def test_in_flight_workspace_is_not_reused():
    pool, made = make_pool()
    first = pool.acquire(KEY, "s0")
    second = pool.acquire(KEY, "s0")
    assert second.buffer is not first.buffer and len(made) == 2
    assert pool.stats.in_flight_bytes == 4096
    done = QueryOnly(ready=False)
    first.release(completion=done)                      # released, not complete, no wait_stream: stays busy
    third = pool.acquire(KEY, "s0")
    assert third.buffer is not first.buffer and len(made) == 3
    done.ready = True
    assert pool.acquire(KEY, "s0").buffer is first.buffer


def test_pending_workspace_is_handed_off_with_stream_ordering():
    pool, made = make_pool()
    lease = pool.acquire(KEY, "producer")
    pending = Completion(ready=False)
    lease.release(completion=pending)
    assert pool.stats.in_flight_bytes == 2048
    taken = pool.acquire(KEY, "consumer")
    assert taken.buffer is lease.buffer and pending.waited == ["consumer"] and len(made) == 1
    assert taken.buffer.recorded_streams == ["producer", "consumer"]
    stats = pool.stats
    assert (stats.hits, stats.misses, stats.in_flight_bytes, stats.cached_bytes) == (1, 1, 2048, 0)
    # the adopted buffer is owned by the new lease only: a later acquire must not adopt it again
    assert pool.acquire(KEY, "other").buffer is not lease.buffer


def test_lru_eviction_over_byte_and_entry_budgets_only_touches_idle_buffers():
    pool, made = make_pool(max_cached_bytes=4096)
    keys = [replace(KEY, chunk_config=(i,)) for i in range(3)]
    leases = [pool.acquire(k, "s") for k in keys]
    for lease in leases:
        lease.release(completion=Completion(ready=True))
    stats = pool.stats
    assert stats.evictions == 1 and stats.cached_bytes == 4096
    pool.acquire(keys[0], "s")                            # the oldest was evicted: allocates again
    assert len(made) == 4
    assert pool.acquire(keys[2], "s").buffer is leases[2].buffer
    entries, _ = make_pool(max_entries=1)
    a, b = entries.acquire(keys[0], "s"), entries.acquire(keys[1], "s")
    a.release(completion=Completion(True))
    b.release(completion=Completion(True))
    assert entries.stats.evictions == 1 and entries.stats.cached_bytes == 2048


def test_zero_budget_never_caches():
    pool, made = make_pool(max_cached_bytes=0)
    pool.acquire(KEY, "s").release(completion=Completion(True))
    assert pool.stats.cached_bytes == 0 and pool.stats.evictions == 1
    pool.acquire(KEY, "s")
    assert len(made) == 2


def test_clear_drops_idle_buffers_only():
    pool, made = make_pool()
    held = pool.acquire(KEY, "s")
    pool.acquire(KEY, "s").release(completion=Completion(True))
    pool.clear()
    assert pool.stats.cached_bytes == 0 and pool.stats.in_flight_bytes == 2048
    held.release(completion=Completion(True))
    assert pool.acquire(KEY, "s").buffer is held.buffer


def test_release_contract():
    pool, _ = make_pool()
    lease = pool.acquire(KEY, "s")
    assert lease.released is False and lease.key == KEY and lease.size_bytes == 2048
    with pytest.raises(TypeError, match="query"):
        lease.release(completion=object())
    assert lease.released is False                        # a failed release can be retried
    lease.release(completion=Completion(True))
    assert lease.released is True
    with pytest.raises(RuntimeError, match="already released"):
        lease.release(completion=Completion(True))
    other, _ = make_pool()
    foreign = WorkspaceLease(other, pool.acquire(KEY, "s")._slot)
    with pytest.raises(RuntimeError, match="not owned by this pool"):
        foreign.release(completion=Completion(True))


def test_concurrent_double_release_enters_the_pool_once():
    pool, _ = make_pool()
    lease = pool.acquire(KEY, "s")
    barrier = threading.Barrier(8)
    outcomes = []

    def worker():
        barrier.wait()
        try:
            lease.release(completion=Completion(True))
            outcomes.append("ok")
        except RuntimeError:
            outcomes.append("dup")

    threads = [threading.Thread(target=worker) for _ in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert sorted(outcomes) == ["dup"] * 7 + ["ok"]
    assert pool.stats.cached_bytes == 2048


# --------------------------------------------------------------------------- #
# output lease
# --------------------------------------------------------------------------- #
class Manager:
    def __init__(self, ready=False):
        self.recorded = []
        self.ready = ready

    def record_for(self, value, *, stream=None):
        self.recorded.append((value, stream))
        return Completion(self.ready)


class Work:
    def __init__(self, done=True):
        self.done = done

    def query(self):
        return self.done


def test_output_lease_life_cycle_and_stream_safe_reuse():
    pool, made = make_pool()
    owner, manager = object(), Manager()
    key = replace(KEY, workspace_kind="reduced_output")
    lease = HipOutputLease(pool.acquire(key, "acquire"), owner_token=owner, completion_manager=manager,
                           acquisition_stream="acquire")
    assert lease.mark_used(owner) is lease.buffer
    lease.bind_work(owner, Work())
    lease.release_after(lease.buffer)
    assert manager.recorded == [(lease.buffer, None)] and len(made) == 1
    assert pool.stats.in_flight_bytes == key.estimated_bytes          # completion still pending
    again = pool.acquire(key, "consumer")
    assert again.buffer is lease.buffer and again.buffer.recorded_streams == ["acquire", "consumer"]


def test_output_lease_rejects_wrong_owner_wrong_order_and_double_release():
    pool, _ = make_pool()
    owner = object()
    lease = HipOutputLease(pool.acquire(KEY, "s0"), owner_token=owner, completion_manager=Manager(),
                           acquisition_stream="s0")
    with pytest.raises(RuntimeError, match="different executor"):
        lease.mark_used(object())
    with pytest.raises(RuntimeError, match="marked used before"):
        lease.release_after(Completion(True))
    lease.mark_used(owner)
    with pytest.raises(RuntimeError, match="after mark_used"):
        lease.release_unused()
    with pytest.raises(RuntimeError, match="already in use"):
        lease.mark_used(owner)
    with pytest.raises(RuntimeError, match="bound to work"):
        lease.release_after(Completion(True))
    lease.abort_use(owner)
    lease.mark_used(owner)
    lease.bind_work(owner, Work(done=False))
    with pytest.raises(RuntimeError, match="until associated work completes"):
        lease.release_after(Completion(True))
    lease._work.done = True
    lease.release_after(Completion(True))
    for call in (lambda: lease.release_after(Completion(True)), lease.release_unused, lambda: lease.mark_used(owner)):
        with pytest.raises(RuntimeError, match="already released"):
            call()


def test_output_lease_unused_release_is_ordered_on_the_acquisition_stream():
    pool, _ = make_pool()
    manager = Manager(ready=True)
    lease = HipOutputLease(pool.acquire(KEY, "acq"), owner_token=object(), completion_manager=manager,
                           acquisition_stream="acq")
    lease.release_unused()
    assert manager.recorded == [(lease.buffer, "acq")] and pool.stats.cached_bytes == 2048
    with pytest.raises(TypeError, match="owner_token must not be None"):
        HipOutputLease(pool.acquire(KEY, "s"), owner_token=None, completion_manager=manager, acquisition_stream="s")
    with pytest.raises(TypeError, match="completion_manager must not be None"):
        HipOutputLease(pool.acquire(KEY, "s"), owner_token=1, completion_manager=None, acquisition_stream="s")
    with pytest.raises(TypeError, match="WorkspaceLease"):
        HipOutputLease(object(), owner_token=1, completion_manager=manager, acquisition_stream="s")

    class Broken:
        def record_for(self, value, *, stream=None):
            raise TypeError("stream completion failed")

    failing = HipOutputLease(pool.acquire(KEY, "s"), owner_token=1, completion_manager=Broken(), acquisition_stream="s")
    with pytest.raises(TypeError, match="stream completion failed"):
        failing.release_unused()
    failing._manager = manager                             # state was restored: the release can be retried
    failing.release_unused()


# --------------------------------------------------------------------------- #
# shard sessions
# --------------------------------------------------------------------------- #
class FakeTensor:
    def __init__(self, numel, dtype="torch.float32"):
        self._numel, self.dtype, self.shape = numel, dtype, (numel,)

    def numel(self):
        return self._numel


def test_shard_session_reuses_send_recv_and_reduced_buffers():
    pool, made = make_pool()
    provider = ShardWorkspaceProvider(pool, backend="hip", collective="reduce_scatter", strategy="compressed",
                                      device="cuda:0")
    cfg = CompressionConfig()
    chunk = FakeTensor(128)
    for step in range(3):
        session = provider.begin(stream="s")
        send = [session.get_quantized_chunk("b", i, chunk, cfg, dtype="fp32", world_size=2) for i in range(2)]
        recv = [session.get_received_tensor_payload("b", i, chunk, cfg, dtype="fp32", world_size=2) for i in range(2)]
        reduced = session.get_reduced_shard("b", chunk, (100,), cfg, dtype="fp32", world_size=2, rank=1)
        assert send[0].key.shape_class == (136,) and send[0].key.workspace_kind == "send"
        assert recv[0].key.workspace_kind == "recv" and recv[0].key.chunk_config == (0, 128)
        assert reduced.key.shape_class == (128,) and reduced.key.chunk_config == (1,)
        assert len(session.leases) == 5
        session.release(completion=Completion(True))
        assert session.leases == ()
    assert len(made) == 5 and pool.stats.hits == 10
    unpooled = ShardWorkspaceProvider(pool, backend="hip", collective="reduce_scatter", strategy="compressed",
                                      device="cuda:0", pool_reduced_output=False)
    assert unpooled.begin(stream="s").get_reduced_shard("b", chunk, (100,), cfg, dtype="fp32", world_size=2,
                                                         rank=0) is None
    with pytest.raises(TypeError, match="pool"):
        ShardWorkspaceProvider(object(), backend="hip", collective="c", strategy="s", device="cuda")


def test_a_released_buffer_nobody_adopts_is_settled_by_the_pool_itself():
    """A completion whose ``peek()`` only turns true after someone has asked ``query()`` (the stream-ordered kind:
    no event until it is needed) must not keep its buffer out of the idle set for ever: after a few polls the pool
    asks the real question once, the buffer becomes idle, and the LRU limits see it."""
    from lowbit_comm_amd.hip import workspace as ws

    class Lazy:
        """No event until query() is called; that call records it and finds it unfinished, every later look finds it
        finished."""

        def __init__(self):
            self.queries = self.peeks = 0

        def peek(self):
            self.peeks += 1
            return self.queries >= 1

        def query(self):
            self.queries += 1
            return self.queries >= 2

    made = []
    pool = ws.HipWorkspacePool(allocator=lambda key, stream: made.append(key) or bytearray(64), max_entries=2)
    keys = [ws.WorkspaceKey(backend="hip", collective="rs", strategy="s", shape_class=(64,), dtype="uint8", world_size=8,
                            bit=8, group_size=64, chunk_config=(i,), workspace_kind="send", device="cpu") for i in range(12)]
    completions = []
    for key in keys[:4]:                        # four shapes that never come back
        lease = pool.acquire(key, None)
        completions.append(Lazy())
        lease.release(completion=completions[-1])
    assert pool.stats.in_flight_bytes == 4 * 64 and pool.stats.cached_bytes == 0
    for key in keys[4:]:                        # other traffic: every acquire polls the pending ones
        pool.acquire(key, None)
    stats = pool.stats
    assert all(c.queries == 1 for c in completions)              # asked by the pool, once, not by a caller
    assert stats.in_flight_bytes == 8 * 64                       # only the eight live leases
    assert stats.cached_bytes == 2 * 64 and stats.evictions == 2  # the four settled buffers met max_entries=2
    # the usual case pays for no query: released and taken over by the next acquire of the same key
    quick = Lazy()
    lease = pool.acquire(keys[0], None)
    lease.release(completion=quick)
    quick.wait_stream = lambda stream: None
    again = pool.acquire(keys[0], None)
    assert quick.queries == 0 and again.buffer is lease.buffer
