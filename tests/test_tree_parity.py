"""GPU parity of the quantized tree all-reduce: every rank on one device (a host thread per rank, device copies as
the links), through the C ABI, against the CPU oracle's simulation (oracle/ring_np.py: tree_all_reduce).
Bar: every rank's bucket bit-exact."""
import threading

import numpy as np
import pytest
import torch

from oracle import ring_np

pytestmark = pytest.mark.gpu

DTYPES = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


def to_np(t, dtype):
    t = t.detach().cpu().contiguous()
    return t.view(torch.int16).numpy().view(np.uint16).copy() if dtype == "bf16" else t.numpy().copy()


def raw(a):
    return a.view({2: np.uint16, 4: np.uint32}[a.dtype.itemsize])


def tensor_like(n, dtype, seed, device, sigma=1e-3):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(n, generator=gen) * sigma
    if n:
        x = torch.where(torch.rand(n, generator=gen) < 2e-3, torch.randn(n, generator=gen) * 1e-1, x)
    return x.to(DTYPES[dtype]).to(device)


def build_tree(device, world, n, dtype, g, root=0, **options):
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.hip.tree import LoopbackMesh, make_tree_executor

    mesh = LoopbackMesh(world, timeout=60.0)
    config = options.pop("config", None) or CompressionConfig(group_size=g)
    return [make_tree_executor(config=config, dtype=dtype, numel=n, world_size=world, rank=r, root=root,
                               send=mesh.send_for(r), recv=mesh.recv_for(r), device=str(device), **options)
            for r in range(world)]


def run_tree(device, executors, buckets):
    world = len(buckets)
    errors = [None] * world

    def body(rank):
        try:
            torch.cuda.set_device(device)
            assert executors[rank].run(buckets[rank]).wait() is buckets[rank]
        except BaseException as error:      # noqa: BLE001 - reported below
            errors[rank] = error

    threads = [threading.Thread(target=body, args=(r,)) for r in range(world)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(180)
    assert not any(t.is_alive() for t in threads)
    first = next((e for e in errors if e is not None), None)
    if first is not None:
        raise first
    torch.cuda.synchronize()


@pytest.mark.parametrize("mode", ["fused", "separate", "pooled"])
@pytest.mark.parametrize("dtype, world, n, g, root", [("fp32", 2, 64 * 9, 64, 0), ("fp32", 5, 10_007, 64, 0),
                                                     ("fp32", 8, 64 * 333 + 13, 64, 3), ("bf16", 4, 33_333, 32, 1),
                                                     ("fp16", 7, 20_000, 16, 6), ("fp32", 1, 1000, 64, 0),
                                                     ("bf16", 3, 5, 16, 2)])
def test_tree_all_reduce_matches_the_oracle_on_every_rank(hip_device, mode, dtype, world, n, g, root):
    options = {"fused": {}, "separate": {"fuse_steps": False}, "pooled": {"max_plans": 0}}[mode]
    buckets = [tensor_like(n, dtype, 7000 + 13 * r, hip_device, sigma=10.0 ** (r % 3 - 3)) for r in range(world)]
    before = [to_np(b, dtype) for b in buckets]
    executors = build_tree(hip_device, world, n, dtype, g, root, **options)
    run_tree(hip_device, executors, buckets)
    want = ring_np.tree_all_reduce(before, dtype, g, root=root)
    for rank in range(world):
        assert np.array_equal(raw(to_np(buckets[rank], dtype)), raw(want[rank])), (rank, mode, dtype, world, n, g, root)


def test_tree_replays_its_plan_without_allocating_and_launches_once_per_changing_step(hip_device):
    world, n, g = 5, 64 * 500 + 7, 64
    executors = build_tree(hip_device, world, n, "fp32", g)
    buckets = [torch.empty(n, device=hip_device) for _ in range(world)]
    for repeat in range(3):
        for r, bucket in enumerate(buckets):
            bucket.copy_(tensor_like(n, "fp32", 800 + 10 * repeat + r, hip_device))
        before = [to_np(b, "fp32") for b in buckets]
        torch.cuda.synchronize()
        allocated = torch.cuda.memory_allocated(hip_device)
        run_tree(hip_device, executors, buckets)
        if repeat:
            assert torch.cuda.memory_allocated(hip_device) == allocated
        want = ring_np.tree_all_reduce(before, "fp32", g)
        assert all(np.array_equal(raw(to_np(buckets[r], "fp32")), raw(want[r])) for r in range(world))
    # rank 1 (children 4 and 3, parent 0): two receive buffers going up, one coming down, and two send buffers:
    # the payload for its parent and the one payload both children get
    plan = next(iter(executors[1]._runtime.plans.values()))
    assert sorted(k for k in plan if k[0] in ("send", "recv")) == [("recv", 0), ("recv", 1), ("recv", 2), ("send", 0),
                                                                  ("send", 1)]
    assert not any(k[0] == "quantize" for k in plan)          # every payload came out of a fused step


POLICIES = [dict(), dict(compact=True), dict(bit=4, allow_experimental=True), dict(topk=1)]


@pytest.mark.parametrize("policy", POLICIES, ids=lambda p: "-".join(f"{k}={v}" for k, v in p.items()) or "linear8")
@pytest.mark.parametrize("dtype, world, g, root", [("fp32", 5, 64, 0), ("bf16", 6, 32, 4), ("fp16", 3, 16, 1)])
def test_tree_through_the_codec_facade_in_the_cuda_byte_format(hip_device, policy, dtype, world, g, root):
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.hip.loader import load_hip_extension

    status = load_hip_extension(wire_format="native")
    assert status.available, status.reason
    config = CompressionConfig(group_size=g, error_feedback=False, **policy)
    n = g * 211
    buckets = [tensor_like(n, dtype, 8100 + 3 * r, hip_device) for r in range(world)]
    before = [to_np(b, dtype) for b in buckets]
    executors = build_tree(hip_device, world, n, dtype, g, root, config=config, extension_status=status)
    run_tree(hip_device, executors, buckets)
    codec = ring_np.CudaWireCodec(g, bit=config.bit, quant_type=config.quant_type, topk=config.topk,
                                  compact=config.compact)
    want = ring_np.tree_all_reduce(before, dtype, g, codec=codec, root=root)
    for rank in range(world):
        assert np.array_equal(raw(to_np(buckets[rank], dtype)), raw(want[rank])), (rank, policy, dtype)


def test_hook_topology_strategy_picks_ring_or_tree_like_the_reference_compiler(hip_device):
    """Group-aligned chunks -> ring, anything else -> tree; both through the DDP hook on every rank of a loopback
    mesh, both bit-exact against the oracle of the schedule that was picked."""
    from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.hip.ring import PipelinedRingExecutor
    from lowbit_comm_amd.hip.tree import LoopbackMesh, TreeExecutor, make_topology_transport

    class Bucket:
        def __init__(self, tensor):
            self._tensor = tensor

        def buffer(self):
            return self._tensor

        def index(self):
            return 0

    world, g = 4, 64
    config = CompressionConfig(group_size=g, error_feedback=False)
    mesh = LoopbackMesh(world, timeout=60.0)
    transports = [make_topology_transport(world_size=world, rank=r, send=mesh.send_for(r), recv=mesh.recv_for(r))
                  for r in range(world)]
    hooks = [create_ddp_comm_hook(config, dtype="auto", strategy="topology", reduce="mean",
                                  topology_all_reduce=transports[r]) for r in range(world)]
    for n, kind, simulate in ((world * g * 20, PipelinedRingExecutor, ring_np.ring_all_reduce),
                              (world * g * 20 + 8, TreeExecutor, ring_np.tree_all_reduce)):
        buckets = [tensor_like(n, "fp32", 8800 + r + n % 7, hip_device) for r in range(world)]
        before = [to_np(b, "fp32") for b in buckets]
        errors = [None] * world

        def body(rank):
            try:
                torch.cuda.set_device(hip_device)
                hooks[rank](None, Bucket(buckets[rank])).wait()
            except BaseException as error:      # noqa: BLE001
                errors[rank] = error

        threads = [threading.Thread(target=body, args=(r,)) for r in range(world)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(180)
        assert errors == [None] * world, errors
        torch.cuda.synchronize()
        assert all(isinstance(t.executors[(n, "fp32", str(hip_device), g)], kind) for t in transports)
        want = simulate(before, "fp32", g)
        for r in range(world):
            assert np.array_equal(raw(to_np(buckets[r], "fp32")), raw(want[r])), (n, r)
