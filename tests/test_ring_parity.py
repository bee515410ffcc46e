"""GPU parity of the ring-step kernel and of the ring all-reduce built on it, through the C ABI, against the CPU
oracle (oracle/ring_np.py) on the same seeded inputs.  Bar: chunk values, int8 codes and fp32 scales bit-exact."""
import numpy as np
import pytest
import torch

from oracle import ring_np

pytestmark = pytest.mark.gpu

DTYPES = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


@pytest.fixture(scope="module", params=["cached", "stream"])
def ops(request, hip_device):
    from lowbit_comm_amd.hip import ops as hip_ops

    with hip_ops.access_mode(request.param):
        yield hip_ops


def to_np(t: torch.Tensor, dtype: str) -> np.ndarray:
    t = t.detach().cpu().contiguous()
    if dtype == "bf16":
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def raw(a: np.ndarray) -> np.ndarray:
    return a.view({2: np.uint16, 4: np.uint32}[a.dtype.itemsize])


def tensor_like(n, dtype, seed, device, sigma=1e-3):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(n, generator=gen) * sigma
    if n:
        mask = torch.rand(n, generator=gen) < 2e-3
        x = torch.where(mask, torch.randn(n, generator=gen) * 1e-1, x)
    return x.to(DTYPES[dtype]).to(device)


def check_step(ops, device, dtype, g, n, reduce_op, divisor, emit, seed, offset=0):
    incoming = tensor_like(n, "fp32", seed, device)
    received = torch.empty(ops.payload_nbytes(n, g), dtype=torch.uint8, device=device)
    assert ops.quant_pack_payload_into(incoming, received, group_size=g)
    backing = tensor_like(n + offset, dtype, seed + 1, device, sigma=3e-3)
    chunk = backing[offset:]
    before = to_np(chunk, dtype)
    send = torch.full((ops.payload_nbytes(n, g),), 0xAB, dtype=torch.uint8, device=device) if emit else None
    assert ops.ring_step_into(received, chunk, send, group_size=g, reduce_op=reduce_op, divisor=divisor)
    groups = ops.num_groups(n, g)
    r = received.cpu().numpy()
    codes, scales = r[:groups * g].view(np.int8), r[groups * g:].view(np.float32)
    want_chunk, want_payload = ring_np.ring_step((codes, scales), before, dtype, g, reduce_op=reduce_op,
                                                 divisor=divisor, emit=emit)
    what = (dtype, g, n, reduce_op, divisor, emit, offset)
    got = to_np(chunk, dtype)
    assert np.array_equal(raw(got), raw(want_chunk)), what
    if offset:
        assert torch.equal(backing[:offset].cpu(), tensor_like(n + offset, dtype, seed + 1, "cpu", sigma=3e-3)[:offset])
    if emit:
        s = send.cpu().numpy()
        assert np.array_equal(s[:groups * g].view(np.int8), want_payload[0]), what
        assert np.array_equal(s[groups * g:].view(np.uint32), want_payload[1].view(np.uint32)), what
    return chunk, send


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("g", [64, 32, 16])
def test_ring_step_bit_exact(ops, hip_device, dtype, g):
    seed = 100
    for n in (1, g - 1, g, 1000, 4096 * 3, 65_536 + 7, 300_001):
        for reduce_op, divisor in (("sum", 1.0), ("sum", 8.0), ("sum", 3.0), ("none", 1.0)):
            for emit in (True, False):
                seed += 2
                check_step(ops, hip_device, dtype, g, n, reduce_op, divisor, emit, seed)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_ring_step_on_unaligned_chunk_views(ops, hip_device, dtype):
    for offset in (1, 3):
        for n in (4096 * 2 + 5, 64 * 100):
            check_step(ops, hip_device, dtype, 64, n, "sum", 8.0, True, 900 + offset, offset=offset)


def test_ring_step_equals_the_three_separate_launches(ops, hip_device):
    g, n = 64, 1_000_003
    for dtype in ("fp32", "bf16"):
        incoming = tensor_like(n, "fp32", 5, hip_device)
        codes, scales = ops.quant_pack(incoming, group_size=g)
        received = torch.cat([codes.view(torch.uint8), scales.view(torch.uint8)])
        start = tensor_like(n, dtype, 6, hip_device, sigma=2e-3)
        fused_chunk = start.clone()
        send = torch.empty_like(received)
        assert ops.ring_step_into(received, fused_chunk, send, group_size=g, reduce_op="sum", divisor=3.0)
        plain = start.clone()
        assert ops.dequant_into(codes, scales, plain, group_size=g, reduce_op="sum")
        ops.true_divide_(plain, 3.0)
        two_codes, two_scales = ops.quant_pack(plain, group_size=g)
        assert torch.equal(fused_chunk.view(torch.int16 if dtype == "bf16" else torch.int32),
                           plain.view(torch.int16 if dtype == "bf16" else torch.int32))
        groups = ops.num_groups(n, g)
        assert torch.equal(send[:groups * g].view(torch.int8), two_codes)
        assert torch.equal(send[groups * g:].view(torch.int32), two_scales.view(torch.int32))


def test_ring_step_special_values(ops, hip_device):
    """NaN and Inf travel as they do through decode, add and quantize: the scale keeps them, codes follow the
    oracle's policy for non-finite quotients."""
    g, n = 64, 64 * 6
    incoming = torch.zeros(n, device=hip_device)
    incoming[5] = 3.0
    received = torch.empty(ops.payload_nbytes(n, g), dtype=torch.uint8, device=hip_device)
    assert ops.quant_pack_payload_into(incoming, received, group_size=g)
    chunk = torch.zeros(n, device=hip_device)
    chunk[70] = float("nan")
    chunk[130] = float("inf")
    chunk[200] = -float("inf")
    chunk[201] = 1.0
    chunk[64 * 4:64 * 5] = 0.0                 # an all-zero group keeps the eps scale
    before = chunk.cpu().numpy().copy()
    send = torch.empty_like(received)
    assert ops.ring_step_into(received, chunk, send, group_size=g, reduce_op="sum")
    r = received.cpu().numpy()
    want_chunk, (want_codes, want_scales) = ring_np.ring_step((r[:n].view(np.int8), r[n:].view(np.float32)), before,
                                                              "fp32", g)
    assert np.array_equal(chunk.cpu().numpy().view(np.uint32), want_chunk.view(np.uint32))
    s = send.cpu().numpy()
    assert np.array_equal(s[n:].view(np.uint32), want_scales.view(np.uint32))
    finite_groups = np.isfinite(want_scales)
    mask = np.repeat(finite_groups, g)
    assert np.array_equal(s[:n].view(np.int8)[mask], want_codes[mask])


def test_ring_step_contract(ops, hip_device):
    g, n = 64, 640
    x = tensor_like(n, "fp32", 1, hip_device)
    received = torch.empty(ops.payload_nbytes(n, g), dtype=torch.uint8, device=hip_device)
    assert ops.quant_pack_payload_into(x, received)
    chunk = torch.zeros(n, device=hip_device)
    assert ops.ring_step_into(received, chunk, None, reduce_op="max") is False            # unsupported, not an error
    odd = torch.zeros(ops.payload_nbytes(n, 48), dtype=torch.uint8, device=hip_device)
    assert ops.ring_step_into(odd, chunk, None, group_size=48) is False
    with pytest.raises(RuntimeError, match="divisor must be > 0"):
        ops.ring_step_into(received, chunk, None, divisor=0.0)
    with pytest.raises(RuntimeError, match="invalid quantized payload size"):
        ops.ring_step_into(received[:-4], chunk, None)
    with pytest.raises(RuntimeError, match="must not alias"):
        ops.ring_step_into(received, chunk, received)
    with pytest.raises(RuntimeError, match="must be a GPU tensor"):
        ops.ring_step_into(received.cpu(), chunk, None)
    with pytest.raises(RuntimeError, match="fp16, bf16 or fp32"):
        ops.ring_step_into(received, chunk.double(), None)
    empty = torch.zeros(0, device=hip_device)
    nothing = torch.zeros(0, dtype=torch.uint8, device=hip_device)
    assert ops.ring_step_into(nothing, empty, nothing.clone())


def test_ring_step_at_the_config4_chunk_size_keeps_the_sum_property(ops, hip_device):
    """6,553,600-element chunk (one eighth of a 200 MiB fp32 bucket): too large for the oracle in seconds, so
    check what must hold at any size: the updated chunk equals the separate decode-accumulate, and the payload
    decodes to within half a scale of it."""
    g, n = 64, 6_553_600
    incoming = tensor_like(n, "fp32", 77, hip_device)
    codes, scales = ops.quant_pack(incoming, group_size=g)
    received = torch.cat([codes.view(torch.uint8), scales.view(torch.uint8)])
    start = tensor_like(n, "fp32", 78, hip_device)
    chunk = start.clone()
    send = torch.empty_like(received)
    assert ops.ring_step_into(received, chunk, send, group_size=g, reduce_op="sum", divisor=8.0)
    plain = start.clone()
    assert ops.dequant_into(codes, scales, plain, group_size=g, reduce_op="sum")
    plain /= 8.0
    assert torch.equal(chunk.view(torch.int32), plain.view(torch.int32))
    out_codes, out_scales = send[:n].view(torch.int8), send[n:].view(torch.float32)
    decoded = out_codes.float().view(-1, g) * out_scales[:, None]
    assert bool(((decoded - chunk.view(-1, g)).abs() <= out_scales[:, None] * 0.5001).all())
    assert int(out_codes.abs().view(-1, g).amax(dim=1).min()) == 127


# --------------------------------------------------------------------------- #
# the whole ring: every rank on one device, one host thread per rank
# --------------------------------------------------------------------------- #
def build_ring(device, world, n, dtype, g, fuse_steps, pools=None, max_plans=16, config=None, extension_status=None):
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.hip.ring import LoopbackRing, make_pipelined_ring_executor

    fabric = LoopbackRing(world, timeout=60.0)
    config = config or CompressionConfig(group_size=g)
    executors = [make_pipelined_ring_executor(config=config, dtype=dtype, numel=n, world_size=world, rank=r,
                                              exchange=fabric.exchange_for(r), fuse_steps=fuse_steps,
                                              pool=None if pools is None else pools[r], device=str(device),
                                              max_plans=max_plans, extension_status=extension_status)
                 for r in range(world)]
    return fabric, executors


def run_ring(device, buckets, dtype, g, fuse_steps, pools=None, max_plans=16, ring=None):
    import threading

    world = len(buckets)
    fabric, executors = ring or build_ring(device, world, buckets[0].numel(), dtype, g, fuse_steps, pools, max_plans)
    errors = [None] * world
    works = [None] * world

    def body(rank):
        try:
            torch.cuda.set_device(device)
            works[rank] = executors[rank].run(buckets[rank])
            assert works[rank].wait() is buckets[rank]
        except BaseException as error:      # noqa: BLE001 - reported by the caller
            errors[rank] = error
            fabric.abort()

    threads = [threading.Thread(target=body, args=(r,)) for r in range(world)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not any(t.is_alive() for t in threads)
    first = next((e for e in errors if e is not None), None)
    if first is not None:
        raise first
    torch.cuda.synchronize()
    return executors, works


@pytest.mark.parametrize("fuse_steps", [True, False])
@pytest.mark.parametrize("dtype, world, n, g", [("fp32", 2, 64 * 9, 64), ("fp32", 3, 10_007, 64), ("fp32", 8, 8 * 64 * 40 + 13, 64),
                                               ("bf16", 4, 33_333, 32), ("fp16", 5, 20_000, 16), ("fp32", 8, 5, 16),
                                               ("bf16", 8, 200_003, 64), ("fp32", 1, 1000, 64)])
@pytest.mark.parametrize("max_plans", [16, 0])
def test_ring_all_reduce_matches_the_oracle_on_every_rank(ops, hip_device, fuse_steps, max_plans, dtype, world, n, g):
    buckets = [tensor_like(n, dtype, 4000 + 17 * r, hip_device, sigma=10.0 ** (r % 3 - 3)) for r in range(world)]
    before = [to_np(b, dtype) for b in buckets]
    run_ring(hip_device, buckets, dtype, g, fuse_steps, max_plans=max_plans)
    want = ring_np.ring_all_reduce(before, dtype, g)
    for rank in range(world):
        got = to_np(buckets[rank], dtype)
        assert np.array_equal(raw(got), raw(want[rank])), (rank, dtype, world, n, g, fuse_steps)


def test_ring_reuses_pooled_workspaces_and_launches_one_kernel_per_hop(ops, hip_device):
    from lowbit_comm_amd.hip.workspace import create_torch_workspace_pool

    world, n, g = 4, 64 * 1000, 64
    pools = [create_torch_workspace_pool() for _ in range(world)]
    results = []
    for repeat in range(3):
        buckets = [tensor_like(n, "fp32", 70 + r, hip_device) for r in range(world)]
        before = [to_np(b, "fp32") for b in buckets]
        executors, _ = run_ring(hip_device, buckets, "fp32", g, True, pools=pools, max_plans=0)
        want = ring_np.ring_all_reduce(before, "fp32", g)
        assert all(np.array_equal(raw(to_np(buckets[r], "fp32")), raw(want[r])) for r in range(world))
        results.append([p.stats for p in pools])
    # 2(W-1) send and 2(W-1) receive buffers per rank, all allocated by the first run
    first, last = results[0], results[-1]
    for rank in range(world):
        assert first[rank].misses == 4 * (world - 1)
        assert last[rank].misses == first[rank].misses
        assert last[rank].hits == 2 * first[rank].misses


@pytest.mark.parametrize("fuse_steps", [True, False])
def test_ring_replays_a_buckets_plan_without_allocating(ops, hip_device, fuse_steps):
    world, n, g = 4, 64 * 777 + 5, 64
    ring = build_ring(hip_device, world, n, "bf16", g, fuse_steps)
    buckets = [torch.empty(n, dtype=torch.bfloat16, device=hip_device) for _ in range(world)]
    other = [torch.empty(n // 2, dtype=torch.bfloat16, device=hip_device) for _ in range(world)]
    allocated = None
    for repeat in range(4):
        fresh = [tensor_like(n, "bf16", 300 + 10 * repeat + r, hip_device) for r in range(world)]
        for bucket, values in zip(buckets, fresh):
            bucket.copy_(values)
        before = [to_np(b, "bf16") for b in buckets]
        del fresh
        torch.cuda.synchronize()
        if repeat >= 1:
            allocated = torch.cuda.memory_allocated(hip_device)
        executors, _ = run_ring(hip_device, buckets, "bf16", g, fuse_steps, ring=ring)
        if repeat >= 1:
            assert torch.cuda.memory_allocated(hip_device) == allocated
        want = ring_np.ring_all_reduce(before, "bf16", g)
        for rank in range(world):
            assert np.array_equal(to_np(buckets[rank], "bf16"), want[rank]), (repeat, rank)
    assert all(len(e._runtime.plans) == 1 for e in ring[1])
    # runs two to four did not go through the per-hop protocol: they replayed the launches the first run recorded
    for e in ring[1]:
        (plan,) = e._runtime.plans.values()
        kinds = [op[0] for op in plan["program"]]
        assert kinds.count("exchange") == 2 * (world - 1)
        assert kinds.count("launch") == (1 + 2 * (world - 1) if fuse_steps else 4 * (world - 1))
    # a second bucket shape gets its own plan; the oldest plan goes when the limit is reached
    for e in ring[1]:
        e._runtime.max_plans = 1
    for bucket in other:
        bucket.normal_(std=1e-3)
    before = [to_np(b, "bf16") for b in other]
    from lowbit_comm_amd.hip.chunk_plan import compile_chunk_plan
    from lowbit_comm_amd.hip.ring import PipelinedRingExecutor, compile_pipelined_ring_schedule

    half_plan = compile_chunk_plan(original_numel=n // 2, world_size=world)
    ring2 = (ring[0], [PipelinedRingExecutor(schedule=compile_pipelined_ring_schedule(chunk_plan=half_plan, rank=r),
                                             runtime=ring[1][r]._runtime, workspace_session_factory=ring[1][r]._sessions,
                                             completion_manager=ring[1][r]._works) for r in range(world)])
    run_ring(hip_device, other, "bf16", g, fuse_steps, ring=ring2)
    want = ring_np.ring_all_reduce(before, "bf16", g)
    for rank in range(world):
        assert np.array_equal(to_np(other[rank], "bf16"), want[rank])
    assert all(list(e._runtime.plans) == [(other[r].data_ptr(), n // 2)] for r, e in enumerate(ring2[1]))


def test_ddp_hook_over_the_ring_transport(ops, hip_device):
    """``create_ddp_comm_hook(strategy="topology", topology_all_reduce=make_pipelined_ring_transport(...))`` on
    every rank of a loopback ring: each rank's bucket ends as the oracle's result for that rank, in place, and a
    second step replays the same executor and plan."""
    import threading

    from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.exceptions import UnsupportedCollective
    from lowbit_comm_amd.hip.ring import LoopbackRing, make_pipelined_ring_transport

    class Bucket:
        def __init__(self, tensor, index=0):
            self._tensor, self._index = tensor, index

        def buffer(self):
            return self._tensor

        def index(self):
            return self._index

    world, n, g = 4, 64 * 500 + 9, 64
    config = CompressionConfig(group_size=g, error_feedback=False)
    fabric = LoopbackRing(world, timeout=60.0)
    transports = [make_pipelined_ring_transport(world_size=world, rank=r, exchange=fabric.exchange_for(r))
                  for r in range(world)]
    hooks = [create_ddp_comm_hook(config, dtype="auto", strategy="topology", reduce="mean",
                                  topology_all_reduce=transports[r]) for r in range(world)]
    assert hooks[0]._ccdl_effective_strategy == "topology"
    buckets = [torch.empty(n, device=hip_device) for _ in range(world)]
    for step in range(2):
        for r, bucket in enumerate(buckets):
            bucket.copy_(tensor_like(n, "fp32", 600 + 10 * step + r, hip_device))
        before = [to_np(b, "fp32") for b in buckets]
        results, errors = [None] * world, [None] * world

        def body(rank):
            try:
                torch.cuda.set_device(hip_device)
                results[rank] = hooks[rank](None, Bucket(buckets[rank], index=3)).wait()
            except BaseException as error:      # noqa: BLE001
                errors[rank] = error
                fabric.abort()

        threads = [threading.Thread(target=body, args=(r,)) for r in range(world)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(120)
        assert not any(t.is_alive() for t in threads)
        assert errors == [None] * world, errors
        torch.cuda.synchronize()
        want = ring_np.ring_all_reduce(before, "fp32", g)
        for r in range(world):
            value = results[r][0] if isinstance(results[r], (list, tuple)) else results[r]
            assert value.data_ptr() == buckets[r].data_ptr()
            assert np.array_equal(raw(to_np(buckets[r], "fp32")), raw(want[r])), (step, r)
    assert all(len(t.executors) == 1 for t in transports)
    with pytest.raises(UnsupportedCollective, match="computes the mean"):
        transports[0](buckets[0], config=config, op="sum")


def test_ring_step_on_more_than_2_to_the_31_elements(hip_device):
    """Indexing is 64-bit: a 4.3 GB bf16 chunk with a ragged tail; group-aligned windows at the start, across the
    2^31 boundary and at the tail are compared with the oracle (a ring step is local to a group)."""
    from lowbit_comm_amd.hip import ops

    g = 64
    n = (1 << 31) + g * 1000 + 5
    chunk = torch.empty(n, dtype=torch.bfloat16, device=hip_device)
    incoming = torch.empty(n, dtype=torch.bfloat16, device=hip_device)
    step = 1 << 28
    for i, a in enumerate(range(0, n, step)):
        b = min(a + step, n)
        gen = torch.Generator(device=hip_device).manual_seed(777 + i)
        chunk[a:b] = (torch.randn(b - a, generator=gen, device=hip_device) * 2e-3).to(torch.bfloat16)
        incoming[a:b] = (torch.randn(b - a, generator=gen, device=hip_device) * 1e-3).to(torch.bfloat16)
    groups = ops.num_groups(n, g)
    received = torch.empty(ops.payload_nbytes(n, g), dtype=torch.uint8, device=hip_device)
    assert ops.quant_pack_payload_into(incoming, received, group_size=g)
    del incoming
    windows = [(0, 1 << 20), ((1 << 31) - g * 2000, (1 << 31) + g * 500), (n - g * 3000 - 5, n)]
    before = [to_np(chunk[a:b], "bf16") for a, b in windows]
    send = torch.empty_like(received)
    assert ops.ring_step_into(received, chunk, send, group_size=g, reduce_op="sum", divisor=3.0)
    torch.cuda.synchronize()
    for (a, b), old in zip(windows, before):
        assert a % g == 0
        first, count = a // g, ops.num_groups(b - a, g)
        codes = received[a:a + count * g].cpu().numpy().view(np.int8)
        scales = received[groups * g + 4 * first:groups * g + 4 * (first + count)].cpu().numpy().view(np.float32)
        want, (w_codes, w_scales) = ring_np.ring_step((codes, scales), old, "bf16", g, reduce_op="sum", divisor=3.0)
        assert np.array_equal(to_np(chunk[a:b], "bf16"), want), (a, b)
        assert np.array_equal(send[a:a + count * g].cpu().numpy().view(np.int8), w_codes), (a, b)
        got_scales = send[groups * g + 4 * first:groups * g + 4 * (first + count)].cpu().numpy().view(np.uint32)
        assert np.array_equal(got_scales, w_scales.view(np.uint32)), (a, b)


POLICIES = [dict(), dict(compact=True), dict(bit=4, allow_experimental=True), dict(topk=2),
            dict(bit=4, quant_type="normal", allow_experimental=True)]


@pytest.mark.parametrize("policy", POLICIES, ids=lambda p: "-".join(f"{k}={v}" for k, v in p.items()) or "linear8")
@pytest.mark.parametrize("dtype, world, g", [("fp32", 4, 64), ("bf16", 3, 32), ("fp16", 8, 16)])
def test_ring_through_the_codec_facade_in_the_cuda_byte_format(hip_device, policy, dtype, world, g):
    """The runtime's facade mode over the module that speaks the CUDA extension's bytes: every hop is the
    reference's own sequence of calls, for policies the ring-step kernel does not serve; every rank's bucket
    equals the oracle's ring over the CUDA-format codec, bit for bit."""
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.hip.loader import load_hip_extension

    status = load_hip_extension(wire_format="native")
    assert status.available, status.reason
    config = CompressionConfig(group_size=g, error_feedback=False, **policy)
    n = world * g * 37
    buckets = [tensor_like(n, dtype, 9100 + 3 * r, hip_device, sigma=10.0 ** (r % 2 - 3)) for r in range(world)]
    before = [to_np(b, dtype) for b in buckets]
    plain = config.bit == 8 and config.topk == 0 and config.quant_type == "linear"
    ring = build_ring(hip_device, world, n, dtype, g, True, config=config, extension_status=status)
    # plain linear codes take the format's own fused step, everything else the module's facade
    assert all(e._runtime._wire_direct is plain and e._runtime._facade is (not plain) for e in ring[1])
    run_ring(hip_device, buckets, dtype, g, True, ring=ring)
    if plain:       # and the facade gives the same bits for them
        again = [torch.from_numpy(b.view(np.int16) if dtype == "bf16" else b).to(hip_device) for b in before]
        again = [a.view(torch.bfloat16) if dtype == "bf16" else a for a in again]
        slow = build_ring(hip_device, world, n, dtype, g, False, config=config, extension_status=status)
        assert all(e._runtime._facade for e in slow[1])
        run_ring(hip_device, again, dtype, g, False, ring=slow)
        for a, b in zip(again, buckets):
            assert np.array_equal(raw(to_np(a, dtype)), raw(to_np(b, dtype)))
    codec = ring_np.CudaWireCodec(g, bit=config.bit, quant_type=config.quant_type, topk=config.topk,
                                  compact=config.compact)
    want = ring_np.ring_all_reduce(before, dtype, g, codec=codec)
    for rank in range(world):
        assert np.array_equal(raw(to_np(buckets[rank], dtype)), raw(want[rank])), (rank, policy, dtype)


def test_ring_through_the_facade_of_the_portable_module_equals_the_fused_ring(hip_device):
    from lowbit_comm_amd.exceptions import UnsupportedCollective
    from lowbit_comm_amd.hip.loader import load_hip_extension

    status = load_hip_extension(wire_format="portable")
    world, g = 3, 64
    n = world * g * 50
    start = [tensor_like(n, "fp32", 9300 + r, hip_device) for r in range(world)]
    fused = [b.clone() for b in start]
    facade = [b.clone() for b in start]
    run_ring(hip_device, fused, "fp32", g, True)
    run_ring(hip_device, facade, "fp32", g, True, ring=build_ring(hip_device, world, n, "fp32", g, True,
                                                                 extension_status=status))
    for a, b in zip(fused, facade):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    ragged = [tensor_like(n + 5, "fp32", 9400 + r, hip_device) for r in range(world)]
    with pytest.raises(UnsupportedCollective, match="group-aligned chunks"):
        run_ring(hip_device, ragged, "fp32", g, True, ring=build_ring(hip_device, world, n + 5, "fp32", g, True,
                                                                      extension_status=status))


def test_ring_step_randomized_sweep(ops, hip_device):
    """Random sizes (ragged, tiny, block-boundary), groups, dtypes, ops, divisors, view offsets; every case
    bit-exact against the oracle.  ``LBC_SWEEP_CASES`` / ``LBC_SWEEP_SEED`` widen or reseed the sweep."""
    import os
    import random

    cases = int(os.environ.get("LBC_SWEEP_CASES", "150"))
    rng = random.Random(int(os.environ.get("LBC_SWEEP_SEED", "2024")))
    edges = [1, 63, 64, 65, 1023, 1024, 4095, 4096, 4097, 8192, 16384, 16385, 65536]
    for case in range(cases):
        dtype = rng.choice(["fp32", "fp16", "bf16"])
        g = rng.choice([16, 32, 64])
        n = rng.choice(edges) + rng.choice([0, 0, 1, -1, 7, 100]) if rng.random() < 0.5 else rng.randint(1, 200_000)
        n = max(1, n)
        reduce_op = rng.choice(["sum", "sum", "none"])
        divisor = rng.choice([1.0, 1.0, 2.0, 3.0, 8.0, 7.0])
        emit = rng.random() < 0.7
        offset = rng.choice([0, 0, 0, 1, 2, 5])
        check_step(ops, hip_device, dtype, g, n, reduce_op, divisor, emit, 50_000 + 3 * case, offset=offset)


@pytest.mark.parametrize("dtype,n", [("fp32", 64 * 8 * 300), ("bf16", 64 * 8 * 101 + 40)])
def test_one_ranks_schedule_replayed_as_a_hip_graph_gives_the_protocols_bits(hip_device, dtype, n):
    """One rank of a W=8 ring with a stand-in for the link that a graph can capture (a device copy of a fixed peer
    payload into the receive buffer).  Run one goes through the per-hop protocol and records, run two captures the
    recorded launches as one graph, runs three and four replay it - with eager work and synchronisations in
    between, and each compared with an executor that only ever uses the protocol."""
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.hip import ops
    from lowbit_comm_amd.hip.ring import make_pipelined_ring_executor

    world, rank, g = 8, 3, 64
    config = CompressionConfig(group_size=g)
    chunk = -(-n // world)
    peer = torch.empty(ops.payload_nbytes(chunk, g), dtype=torch.uint8, device=hip_device)
    assert ops.quant_pack_payload_into(tensor_like(chunk, "fp32", 9100, hip_device), peer)

    class Arrived:
        def query(self):
            return True

        def wait_stream(self, stream):
            return None

    def exchange(payload, received, *, send_peer, recv_peer, stream):
        with torch.cuda.stream(stream):
            received.copy_(peer[:received.numel()], non_blocking=True)
        return Arrived()

    protocol = make_pipelined_ring_executor(config=config, dtype=dtype, numel=n, world_size=world, rank=rank,
                                            exchange=exchange, max_plans=0)
    graphed = make_pipelined_ring_executor(config=config, dtype=dtype, numel=n, world_size=world, rank=rank,
                                           exchange=exchange, graph_replay=True)
    bucket = torch.empty(n, dtype=DTYPES[dtype], device=hip_device)
    for run in range(4):
        values = tensor_like(n, dtype, 9200 + run, hip_device)
        want = values.clone()
        assert protocol.run(want).wait() is want
        bucket.copy_(values)
        assert graphed.run(bucket).wait() is bucket
        torch.cuda.synchronize()
        assert np.array_equal(raw(to_np(bucket, dtype)), raw(to_np(want, dtype))), run
        assert float((torch.randn(1 << 16, device=hip_device) * 2).sum().item()) == pytest.approx(0.0, abs=1e4)   # eager work
    (plan,) = graphed._runtime.plans.values()
    assert isinstance(plan["graph"], torch.cuda.CUDAGraph) and len(plan["program"]) == 1 + 4 * (world - 1)


def test_ring_steps_captured_in_a_hip_graph_replay_like_eager(hip_device):
    """A chain of ring steps (each hop's payload feeds the next) allocates and clears nothing, so it can be captured;
    four replays with eager work and synchronisations in between equal four eager passes from the same state."""
    from lowbit_comm_amd.hip import ops

    g, n, hops = 64, 64 * 3000 + 21, 5
    incoming = torch.empty(ops.payload_nbytes(n, g), dtype=torch.uint8, device=hip_device)
    assert ops.quant_pack_payload_into(tensor_like(n, "fp32", 31, hip_device), incoming, group_size=g)
    start = tensor_like(n, "fp32", 32, hip_device)
    chunks = [start.clone() for _ in range(hops)]
    payloads = [torch.empty_like(incoming) for _ in range(hops)]
    launches = [ops.bind_ring_step(incoming if h == 0 else payloads[h - 1], chunks[h], payloads[h], group_size=g,
                                   reduce_op="sum", divisor=2.0 if h == hops - 1 else 1.0) for h in range(hops)]

    def one_pass():
        for launch in launches:
            assert launch()

    eager = []
    for _ in range(4):
        one_pass()
        torch.cuda.synchronize()
        eager.append(([c.clone() for c in chunks], payloads[-1].clone()))
    for c in chunks:
        c.copy_(start)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
        one_pass()
    torch.cuda.synchronize()
    for c in chunks:
        c.copy_(start)                                               # capture enqueued nothing
    for want_chunks, want_payload in eager:
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a.view(torch.int32), b.view(torch.int32)) for a, b in zip(chunks, want_chunks))
        assert torch.equal(payloads[-1], want_payload)
        assert torch.isfinite((torch.randn(1 << 16, device=hip_device) * 2).sum())   # eager work between replays


# --------------------------------------------------------------------------- #
# the same hop in the CUDA extension's byte format
# --------------------------------------------------------------------------- #
def check_wire_step(device, dtype, g, n, compact, reduce_op, divisor, emit, seed, poison=False, lead=0, send_lead=0):
    from lowbit_comm_amd.hip import cuda_wire

    tdtype = DTYPES[dtype]
    incoming = tensor_like(n, dtype, seed, device)
    received = cuda_wire.quant_pack(incoming, group_size=g, compact=compact)
    if lead:                                      # the payload at a 2-byte aligned address, other bytes after it
        holder = torch.full((received.numel() + lead + 16,), 0x5A, dtype=torch.uint8, device=device)
        holder[lead:lead + received.numel()].copy_(received)
        received = holder[lead:lead + received.numel()]
    chunk = tensor_like(n, dtype, seed + 1, device, sigma=3e-3)
    if poison and n >= 4 * g:
        chunk[g + 3] = float("nan")               # a NaN inside a group: the running maximum restarts after it
        chunk[3 * g - 1] = float("nan")           # a NaN that ends a group's scan
        chunk[5] = float("inf")
    before = to_np(chunk, dtype)
    send = None
    if emit:                                      # send_lead: the outgoing payload at a 2-byte aligned address
        room = torch.full((cuda_wire.payload_nbytes(n, tdtype, g) + send_lead + 16,), 0xAB, dtype=torch.uint8, device=device)
        send = room[send_lead:send_lead + cuda_wire.payload_nbytes(n, tdtype, g)]
    assert cuda_wire.ring_step_into(received, chunk, send, group_size=g, compact=compact, reduce_op=reduce_op,
                                    divisor=divisor)
    codec = ring_np.CudaWireCodec(g, compact=compact)
    want_chunk, want_payload = ring_np.ring_step(received.cpu().numpy(), before, dtype, g, reduce_op=reduce_op,
                                                 divisor=divisor, emit=emit, codec=codec)
    what = (dtype, g, n, compact, reduce_op, divisor, emit, poison)
    assert np.array_equal(raw(to_np(chunk, dtype)), raw(want_chunk)), what
    if emit:
        assert np.array_equal(send.cpu().numpy(), want_payload), what
        assert bool((room[:send_lead] == 0xAB).all()) and bool((room[send_lead + send.numel():] == 0xAB).all()), what


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_wire_gather_hop_of_a_large_chunk_bit_exact(hip_device, dtype):
    """From 4 Mi elements on, the hop that only decodes and requantizes writes a 16-bit payload with interleaved
    scales as whole dwords shifted across lanes.  An odd number of groups (the last group has no partner), an even
    one with NaNs and an infinity in the chunk, and an outgoing payload at a 2-byte aligned address (the kernel's
    other store path at this size); bytes around the payload stay untouched.  Sizes on both sides of the bound."""
    bound = 1 << 16                                    # groups of 64: 4 Mi elements
    check_wire_step(hip_device, dtype, 64, 64 * bound, True, "none", 1.0, True, 80_990)
    check_wire_step(hip_device, dtype, 64, 64 * (bound - 1), True, "none", 1.0, True, 80_992)
    check_wire_step(hip_device, dtype, 64, 64 * (bound + 1), True, "none", 1.0, True, 80_994, poison=True)
    check_wire_step(hip_device, dtype, 64, 64 * (bound + 2), True, "none", 1.0, True, 80_996, lead=2, send_lead=2)
    groups = 1 << 18
    check_wire_step(hip_device, dtype, 64, 64 * (groups + 1), True, "none", 1.0, True, 81_000)
    check_wire_step(hip_device, dtype, 64, 64 * (groups + 2), True, "none", 1.0, True, 81_002, poison=True)
    check_wire_step(hip_device, dtype, 64, 64 * (groups + 3), True, "none", 1.0, True, 81_004, lead=2, send_lead=2)
    check_wire_step(hip_device, dtype, 64, 64 * (groups + 5), True, "sum", 8.0, True, 81_006)


@pytest.mark.parametrize("compact", [True, False])
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_wire_ring_step_bit_exact(hip_device, dtype, compact):
    seed = 70_000
    for g in (64, 32, 16):
        for n in (g, g * 17, g * 4096 // 16 + g, g * 5000):
            for reduce_op, divisor in (("sum", 1.0), ("sum", 8.0), ("sum", 3.0), ("none", 1.0)):
                for emit in (True, False):
                    seed += 2
                    check_wire_step(hip_device, dtype, g, n, compact, reduce_op, divisor, emit, seed)
    check_wire_step(hip_device, dtype, 64, 64 * 40, compact, "sum", 1.0, True, 79_001, poison=True)
    check_wire_step(hip_device, dtype, 16, 16 * 64, compact, "none", 1.0, True, 79_003, poison=False)
    if dtype != "fp32":                            # 66-byte groups: every parity of address and of group count
        for n in (64, 64 * 2, 64 * 3, 64 * 33, 64 * 4096 // 16 + 64):
            for lead in (2, 4, 6):
                for reduce_op in ("none", "sum"):
                    seed += 2
                    check_wire_step(hip_device, dtype, 64, n, compact, reduce_op, 1.0, True, seed, lead=lead)


def test_wire_ring_step_equals_the_separate_launches_and_checks_its_arguments(hip_device):
    from lowbit_comm_amd.hip import cuda_wire

    g, n = 64, 64 * 20_000
    for dtype in (torch.float32, torch.bfloat16):
        received = cuda_wire.quant_pack(tensor_like(n, "fp32", 5, hip_device).to(dtype))
        start = tensor_like(n, "fp32", 6, hip_device).to(dtype)
        fused = start.clone()
        send = torch.empty_like(received)
        assert cuda_wire.ring_step_into(received, fused, send, reduce_op="sum", divisor=3.0)
        plain = start.clone()
        assert cuda_wire.dequant_into(received, plain, reduce_op="sum")
        plain.div_(3)
        assert torch.equal(fused.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                           plain.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
        assert torch.equal(send, cuda_wire.quant_pack(plain))
    chunk = torch.zeros(64 * 3, device=hip_device)
    payload = cuda_wire.quant_pack(chunk)
    assert cuda_wire.ring_step_into(payload, chunk, None, reduce_op="max") is False
    with pytest.raises(RuntimeError, match="multiple of group_size"):
        cuda_wire.ring_step_into(payload, chunk[:100], None)
    with pytest.raises(RuntimeError, match="invalid quantized payload size"):
        cuda_wire.ring_step_into(payload[:-4], chunk, None)
    with pytest.raises(RuntimeError, match="must not alias"):
        cuda_wire.ring_step_into(payload, chunk, payload)
    with pytest.raises(RuntimeError, match="divisor must be > 0"):
        cuda_wire.ring_step_into(payload, chunk, None, divisor=-1.0)
