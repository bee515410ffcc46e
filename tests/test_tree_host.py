"""Host logic of the quantized tree: compiled schedule (properties and the five-rank edge list the reference
states in tests/cuda/test_topology_executors.py:1673-1760), the executor's call order, validation.  CPU only."""
import pytest

from lowbit_comm_amd.hip.chunk_plan import compile_chunk_plan
from lowbit_comm_amd.hip.tree import TreeEdge, TreeExecutor, TreeSchedule, compile_tree_schedule, rank_actions
from oracle import ring_np


@pytest.mark.parametrize("world", [1, 2, 3, 5, 8, 13])
def test_every_root_gives_a_connected_acyclic_tree_that_every_rank_agrees_on(world):
    plan = compile_chunk_plan(original_numel=world * 5, world_size=world)
    for root in range(world):
        at_root = compile_tree_schedule(chunk_plan=plan, rank=root, root=root)
        assert at_root.parent is None and at_root.local_chunk == plan.chunk_for_rank(root)
        assert len(at_root.reduce_edges) == world - 1
        assert at_root.broadcast_edges == tuple(reversed(at_root.reduce_edges))
        assert {e.child_rank for e in at_root.reduce_edges} == set(range(world)) - {root}
        assert [(e.child_rank, e.parent_rank) for e in at_root.reduce_edges] == ring_np.tree_edges(world, root)
        parents = {e.child_rank: e.parent_rank for e in at_root.reduce_edges}
        for child in parents:
            seen, at = set(), child
            while at != root:
                assert at not in seen
                seen.add(at)
                at = parents[at]
        for rank in range(world):
            local = compile_tree_schedule(chunk_plan=plan, rank=rank, root=root)
            assert local.reduce_edges == at_root.reduce_edges
            assert local.parent == parents.get(rank)
            assert local.children == tuple(e.child_rank for e in at_root.reduce_edges if e.parent_rank == rank)


def test_five_ranks_have_the_edges_the_reference_test_names():
    schedule = compile_tree_schedule(chunk_plan=compile_chunk_plan(original_numel=25, world_size=5), rank=1, root=0)
    assert [(e.child_rank, e.parent_rank) for e in schedule.reduce_edges] == [(4, 1), (3, 1), (2, 0), (1, 0)]
    assert schedule.parent == 0 and schedule.children == (4, 3)
    assert [(a, e.child_rank, e.parent_rank) for a, e in rank_actions(schedule)] == [
        ("reduce", 4, 1), ("reduce", 3, 1), ("send_up", 1, 0), ("receive_down", 1, 0), ("send_down", 3, 1),
        ("send_down", 4, 1)]


def test_schedule_and_edges_are_validated():
    plan = compile_chunk_plan(original_numel=25, world_size=5)
    good = compile_tree_schedule(chunk_plan=plan, rank=2, root=1)
    fields = dict(chunk_plan=plan, rank=2, root=1, parent=good.parent, children=good.children,
                  reduce_edges=good.reduce_edges, broadcast_edges=good.broadcast_edges)
    TreeSchedule(**fields)
    for change, text in (({"reduce_edges": good.reduce_edges[::-1]}, "reduce_edges must match"),
                         ({"broadcast_edges": good.reduce_edges}, "broadcast_edges must reverse"),
                         ({"parent": None}, "parent must match"), ({"children": (0,)}, "children must match"),
                         ({"root": 5}, r"root must be in \[0, 5\)")):
        with pytest.raises(ValueError, match=text):
            TreeSchedule(**{**fields, **change})
    with pytest.raises(TypeError, match="chunk_plan must be a ChunkPlan"):
        compile_tree_schedule(chunk_plan=None, rank=0)
    with pytest.raises(ValueError, match="must differ"):
        TreeEdge(child_rank=1, parent_rank=1)
    with pytest.raises(TypeError, match="child_rank must be an integer"):
        TreeEdge(child_rank=1.0, parent_rank=0)


class Endpoint:
    def query(self):
        return False

    def wait(self):
        return None

    def wait_stream(self, stream):
        return None


class Handle:
    def is_completed(self):
        return True


class Runtime:
    def __init__(self):
        self.calls, self.handles = [], []
        self.context, self.completion = Endpoint(), Endpoint()

    def create_submission_context(self, tensor):
        self.calls.append(("create_submission_context", tensor))
        return self.context

    def wait_for_producer(self, tensor, *, context):
        self.calls.append(("producer_wait", tensor))

    def _handle(self):
        self.handles.append(Handle())
        return self.handles[-1]

    def quant_pack(self, tensor, edge, workspace, *, context):
        self.calls.append(("quant_pack", edge, workspace))
        return ("payload", edge)

    def send(self, payload, *, peer, edge, workspace, context):
        self.calls.append(("send", peer, edge, workspace))
        return self._handle()

    def receive(self, *, peer, edge, workspace, context):
        self.calls.append(("receive", peer, edge, workspace))
        return ("received", edge), self._handle()

    def fused_reduce(self, tensor, received, edge, workspace, *, context, dependency):
        assert dependency is self.handles[-1]
        self.calls.append(("fused_reduce", edge, workspace))

    def apply_broadcast(self, tensor, received, edge, workspace, *, context, dependency):
        assert dependency is self.handles[-1]
        self.calls.append(("apply_broadcast", edge, workspace))

    def record_completion(self, *, context, dependencies):
        self.calls.append("record_completion")
        self.dependencies = dependencies
        return self.completion


class Session:
    def __init__(self):
        self.released_with = []

    def release(self, *, completion):
        self.released_with.append(completion)


class Work:
    def __init__(self, result, completion, resources):
        self.result, self.completion, self.resources = result, completion, resources

    def query(self):
        return self.completion.query()


class Works:
    def create_work(self, *, result, completion, resources):
        return Work(result, completion, resources)


def test_executor_reduces_up_then_broadcasts_down_in_edge_order():
    schedule = compile_tree_schedule(chunk_plan=compile_chunk_plan(original_numel=25, world_size=5), rank=1, root=0)
    e41, e31, _e20, e10 = schedule.reduce_edges
    runtime, session, tensor = Runtime(), Session(), object()
    executor = TreeExecutor(schedule=schedule, runtime=runtime, workspace_session_factory=lambda t: session,
                            completion_manager=Works())
    work = executor.run(tensor)
    assert runtime.calls == [
        ("create_submission_context", tensor), ("producer_wait", tensor),
        ("receive", 4, e41, session), ("fused_reduce", e41, session),
        ("receive", 3, e31, session), ("fused_reduce", e31, session),
        ("quant_pack", e10, session), ("send", 0, e10, session),
        ("receive", 0, e10, session), ("apply_broadcast", e10, session),
        ("quant_pack", e31, session), ("send", 3, e31, session),
        ("quant_pack", e41, session), ("send", 4, e41, session),
        "record_completion"]
    assert work.result is tensor and work.query() is False
    assert session in work.resources and all(h in work.resources for h in runtime.handles)
    assert all(h in runtime.dependencies for h in runtime.handles)
    assert session.released_with == [work.completion]
    with pytest.raises(TypeError, match="schedule must be a TreeSchedule"):
        TreeExecutor(schedule=object(), runtime=runtime, workspace_session_factory=lambda t: session,
                     completion_manager=Works())


def test_root_and_leaf_do_only_their_part():
    plan = compile_chunk_plan(original_numel=25, world_size=5)
    root = [a for a, _ in rank_actions(compile_tree_schedule(chunk_plan=plan, rank=0))]
    leaf = [a for a, _ in rank_actions(compile_tree_schedule(chunk_plan=plan, rank=4))]
    assert root == ["reduce", "reduce", "send_down", "send_down"]
    assert leaf == ["send_up", "receive_down"]
    assert rank_actions(compile_tree_schedule(chunk_plan=compile_chunk_plan(original_numel=3, world_size=1), rank=0)) == ()


def test_runtime_precomputes_which_steps_feed_a_send_and_which_completes_the_sum():
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.hip.tree import HipTreeRuntime

    plan = compile_chunk_plan(original_numel=64 * 5, world_size=5)

    def runtime(rank):
        return HipTreeRuntime(schedule=compile_tree_schedule(chunk_plan=plan, rank=rank), config=CompressionConfig(),
                              dtype="fp32", send=lambda *a, **k: None, recv=lambda *a, **k: None)

    root, inner, leaf = runtime(0), runtime(1), runtime(4)
    assert root._sent_next == (False, True) and root._completes_sum == 1
    assert inner._sent_next == (False, True, True) and inner._completes_sum is None
    assert leaf._sent_next == (False,) and leaf._completes_sum is None
    with pytest.raises(TypeError, match="recv must be callable"):
        HipTreeRuntime(schedule=compile_tree_schedule(chunk_plan=plan, rank=0), config=CompressionConfig(),
                       dtype="fp32", send=lambda: None, recv=None)
