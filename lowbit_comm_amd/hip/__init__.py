"""HIP (gfx950) backend: C-ABI binding, tensor-level ops, native-module shim, codec callables, workspace pool."""
from .completion import HipCompletionManager, HipStreamWork
from .lanes import StreamLanes
from .loader import CudaExtensionStatus, HipExtensionStatus, load_cuda_extension, load_hip_extension
from .ring import (
    HipPipelinedRingRuntime,
    JoinedCompletion,
    LoopbackRing,
    PipelinedRingExecutor,
    PipelinedRingSchedule,
    RingAllGatherStep,
    RingReduceScatterStep,
    compile_pipelined_ring_schedule,
    make_pipelined_ring_executor,
)
from .tree import HipTreeRuntime, LoopbackMesh, TreeEdge, TreeExecutor, TreeSchedule, compile_tree_schedule, make_tree_executor
from .workspace import (
    CudaOutputLease,
    CudaShardWorkspaceProvider,
    CudaShardWorkspaceSession,
    CudaWorkspacePool,
    EventCompletion,
    EventCompletionManager,
    HipOutputLease,
    HipWorkspacePool,
    ShardWorkspaceProvider,
    ShardWorkspaceSession,
    StreamOrderedCompletion,
    WorkspaceKey,
    WorkspaceLease,
    WorkspaceStats,
    create_torch_workspace_pool,
)

__all__ = [
    "CudaExtensionStatus", "CudaOutputLease", "CudaShardWorkspaceProvider", "CudaShardWorkspaceSession",
    "CudaWorkspacePool", "EventCompletion", "EventCompletionManager", "HipCompletionManager", "HipExtensionStatus",
    "HipOutputLease", "HipPipelinedRingRuntime", "HipStreamWork", "JoinedCompletion", "LoopbackRing",
    "PipelinedRingExecutor", "PipelinedRingSchedule", "RingAllGatherStep", "RingReduceScatterStep",
    "compile_pipelined_ring_schedule", "make_pipelined_ring_executor", "HipTreeRuntime", "LoopbackMesh", "TreeEdge",
    "TreeExecutor", "TreeSchedule", "compile_tree_schedule", "make_tree_executor",
    "HipWorkspacePool", "ShardWorkspaceProvider", "ShardWorkspaceSession", "StreamLanes", "StreamOrderedCompletion",
    "WorkspaceKey",
    "WorkspaceLease", "WorkspaceStats", "create_torch_workspace_pool", "load_cuda_extension", "load_hip_extension",
]
