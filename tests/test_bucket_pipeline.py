"""GPU tests of the bucket pipeline: a stream of buckets through the pipelined reduce-scatter (+ all-gather) transport
must leave, bit for bit, what the unpipelined transport leaves and what the CPU oracle computes, with one launch per
bucket (counted with torch.profiler), through the transport, through ``compressed_reduce_scatter_shard`` and through
``create_ddp_comm_hook(strategy="reduce_scatter")``.

The exchanges are stand-ins on the one GPU: the all-to-all hands this rank its own W chunk payloads back (as if every
peer had sent what this rank sends to it), the all-gather fills every row with this rank's requantized shard."""
import pytest
import torch

from lowbit_comm_amd import CompressionConfig
from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
from oracle import codec_torch

pytestmark = pytest.mark.gpu
CFG = CompressionConfig()
G = 64
NAMES = {torch.float32: "fp32", torch.bfloat16: "bf16", torch.float16: "fp16"}


def grad(n, dtype, seed, dev, sigma=1e-3):
    gen = torch.Generator().manual_seed(seed)
    return (torch.randn(n, generator=gen) * sigma).to(dtype).to(dev)


def same_bits(a, b):
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    assert a.dtype == b.dtype and a.shape == b.shape, (a.dtype, b.dtype, a.shape, b.shape)
    view = torch.int32 if a.dtype == torch.float32 else torch.int16
    return torch.equal(a.view(view), b.view(view))


def loopback_all_to_all(received, send):
    received.copy_(send)


def loopback_all_gather(gathered, mine):
    gathered[1:, :mine.numel()] = mine             # row 0, this rank's, is in place


def oracle_all_reduce(bucket_cpu, residual_cpu, world, op="mean"):
    """The plan on the CPU for the loopback exchanges: returns (reduced bucket, new residual, reduced shard)."""
    n, name = bucket_cpu.numel(), NAMES[bucket_cpu.dtype]
    shard = -(-n // world)
    prepared = bucket_cpu if residual_cpu is None else bucket_cpu + residual_cpu
    padded = torch.cat([prepared, prepared.new_zeros(shard * world - n)])
    payloads, dropped = [], []
    for d in range(world):
        chunk = padded[d * shard:(d + 1) * shard]
        codes, scales = codec_torch.quantize(chunk, G)
        payloads.append((codes, scales))
        dropped.append(chunk - codec_torch.dequantize(codes, scales, shard, G, "fp32"))
    reduced = codec_torch.reduce_payloads(payloads, shard, G, name, op)
    again = codec_torch.dequantize(*codec_torch.quantize(reduced, G), shard, G, name)
    return again.repeat(world)[:n], torch.cat(dropped)[:n], reduced


class Bucket:
    def __init__(self, tensor, index, last):
        self._tensor, self._index, self._last = tensor, index, last

    def buffer(self):
        return self._tensor

    def index(self):
        return self._index

    def is_last(self):
        return self._last


def transports(world, *, error_feedback, lanes=1):
    from lowbit_comm_amd.hip.reduce_scatter import make_reduce_scatter_transport

    common = dict(world_size=world, rank=0, all_to_all=loopback_all_to_all, all_gather=loopback_all_gather,
                  error_feedback=error_feedback)
    return make_reduce_scatter_transport(pipelined=True, lanes=lanes, **common), make_reduce_scatter_transport(**common)


def kernel_counts(run):
    """Names of the kernels `run` launches, with their counts."""
    from torch.profiler import ProfilerActivity, profile

    torch.cuda.synchronize()
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        run()
        torch.cuda.synchronize()
    counts = {}
    for event in prof.events():
        if event.device_type == torch.autograd.DeviceType.CUDA:
            counts[event.name] = counts.get(event.name, 0) + 1
    return counts


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("error_feedback", [False, True])
@pytest.mark.parametrize("world,lanes", [(8, 1), (8, 2), (4, 1), (2, 3), (6, 1), (3, 2), (1, 1)])
def test_pipelined_transport_equals_the_unpipelined_one_and_the_oracle(hip_device, dtype, error_feedback, world, lanes):
    sizes = [G * world * 40, G * world * 40, G * world * 24, G * world * 40 + 8 * world, 70_001, G * world * 40, 640]
    piped, plain = transports(world, error_feedback=error_feedback, lanes=lanes)
    originals = [grad(n, dtype, 700 + k, hip_device) for k, n in enumerate(sizes)]
    mine = [t.clone() for t in originals]
    theirs = [t.clone() for t in originals]
    cpu_residuals = [None] * len(sizes)
    for step in range(3):                         # three iterations: the residuals carry over, the plans are reused
        for k, original in enumerate(originals):
            fresh = grad(original.numel(), dtype, 900 + 10 * step + k, hip_device)
            mine[k].copy_(fresh)
            theirs[k].copy_(fresh)
        inputs = [t.cpu() for t in mine]
        futures = [piped(t, config=CFG, op="mean") for t in mine]
        assert not futures[-1].done()
        piped.flush()
        results = [f.wait() for f in futures]
        wanted = [plain(t, config=CFG, op="mean") for t in theirs]
        torch.cuda.synchronize()
        for k, (got, want) in enumerate(zip(results, wanted)):
            assert got.data_ptr() == mine[k].data_ptr()                  # decoded in place
            assert same_bits(got, want), f"bucket {k}, step {step}"
            reduced, dropped, _shard = oracle_all_reduce(inputs[k], cpu_residuals[k] if error_feedback else None, world)
            assert same_bits(got, reduced), f"bucket {k}, step {step}, against the oracle"
            if error_feedback:
                cpu_residuals[k] = dropped
        if error_feedback:
            for k in range(len(sizes)):
                key = (mine[k].data_ptr(), mine[k].numel(), mine[k].dtype)
                other = (theirs[k].data_ptr(), theirs[k].numel(), theirs[k].dtype)
                assert same_bits(piped.residuals[key], plain.residuals[other]), f"residual {k}, step {step}"
                assert same_bits(piped.residuals[key], cpu_residuals[k]), f"residual {k}, step {step}, against the oracle"
    stats = piped.pipeline.stats
    assert stats["buckets"] == 3 * len(sizes) and stats["flushes"] == 3
    assert stats["merged_launches"] + stats["separate_launches"] >= stats["buckets"]


def test_one_launch_per_bucket_counted_on_the_device(hip_device):
    world, n, buckets = 8, G * 8 * 400, 12
    piped, plain = transports(world, error_feedback=True)
    tensors = [grad(n, torch.bfloat16, 40 + k, hip_device) for k in range(buckets)]

    def run(transport):
        def go():
            futures = [transport(t, config=CFG, op="mean") for t in tensors]
            transport.flush()
            return futures
        return go

    run(piped)()                                   # plans, residuals and bound launches exist after the first pass
    run(plain)()
    counts = kernel_counts(run(piped))
    codec = {name: c for name, c in counts.items() if "lbc" in name}      # some names arrive mangled (_ZN3lbc...)
    assert codec, sorted(counts)
    steps = sum(c for name, c in codec.items() if "bucket_pipeline_step_kernel" in name)
    assert steps == buckets                        # buckets 1..11 with earlier stages, plus reduce + decode at the flush
    assert sum(codec.values()) == buckets + 2      # the first quantize and the last decode stand alone
    plain_counts = kernel_counts(run(plain))
    assert sum(c for name, c in plain_counts.items() if "lbc" in name) == 3 * buckets


def test_second_iteration_allocates_nothing_and_binds_nothing(hip_device):
    from lowbit_comm_amd.hip import ops

    world, n = 8, G * 8 * 100
    piped, _plain = transports(world, error_feedback=True)
    tensors = [grad(n, torch.bfloat16, 60 + k, hip_device) for k in range(7)]
    for _ in range(2):
        for t in tensors:
            piped(t, config=CFG, op="mean")
        piped.flush()
    torch.cuda.synchronize()
    allocated = torch.cuda.memory_allocated()
    bound = {name: getattr(ops, name) for name in ("bind_quant_pack_chunks", "bind_dequant_reduce_quant",
                                                   "bind_dequant_chunks", "bind_bucket_pipeline_step")}
    calls = []
    try:
        for name, fn in bound.items():
            setattr(ops, name, lambda *a, _fn=fn, _name=name, **k: calls.append(_name) or _fn(*a, **k))
        for t in tensors:
            piped(t, config=CFG, op="mean")
        piped.flush()
    finally:
        for name, fn in bound.items():
            setattr(ops, name, fn)
    torch.cuda.synchronize()
    assert calls == []
    assert torch.cuda.memory_allocated() == allocated


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_reduce_scatter_leg_through_compressed_reduce_scatter_shard(hip_device, dtype):
    """``compressed_reduce_scatter_shard(async_op=True, pipeline=...)``: the quantize of bucket k and the reduce of bucket
    k-1 in one launch; every bucket's shard equals the synchronous call's and the oracle's."""
    from lowbit_comm_amd.communication.async_shard_pipeline import AsyncShardPipeline
    from lowbit_comm_amd.hip.bucket_pipeline import BucketPipeline
    from lowbit_comm_amd.hip.reduce_scatter import compressed_reduce_scatter_shard

    world = 8
    sizes = [G * world * 50, G * world * 50, 33_333, G * world * 50]
    tensors = [grad(n, dtype, 300 + k, hip_device) for k, n in enumerate(sizes)]
    pipe = BucketPipeline(world_size=world, rank=0, all_to_all=loopback_all_to_all)
    order = []
    works = [compressed_reduce_scatter_shard(t, config=CFG, world_size=world, rank=0, all_to_all=loopback_all_to_all,
                                             op="sum", async_op=True, pipeline=pipe,
                                             update_feedback=lambda shard, k=k: order.append(("feedback", k)),
                                             advance_policy=lambda k=k: order.append(("advance", k)))
             for k, t in enumerate(tensors)]
    assert all(isinstance(w, AsyncShardPipeline) for w in works)
    assert [w.query() for w in works] == [True, True, True, False]
    last = works[-1].wait()                                   # waiting flushes the pipeline
    assert pipe.pending == 0 and works[-1].query()
    assert order == [(what, k) for k in range(4) for what in ("feedback", "advance")]
    for k, (work, tensor) in enumerate(zip(works, tensors)):
        shard = work.wait()
        want = compressed_reduce_scatter_shard(tensor, config=CFG, world_size=world, rank=0, all_to_all=loopback_all_to_all, op="sum")
        torch.cuda.synchronize()
        assert shard.metadata["async_completion"] is True and shard.shard_numel == want.shard_numel
        assert same_bits(shard.shard, want.shard), f"bucket {k}"
        _reduced, _dropped, oracle_shard = oracle_all_reduce(tensor.cpu(), None, world, op="sum")
        assert same_bits(shard.shard, oracle_shard), f"bucket {k} against the oracle"
    assert last.shard_index == 0
    counts = kernel_counts(lambda: [compressed_reduce_scatter_shard(
        t, config=CFG, world_size=world, rank=0, all_to_all=loopback_all_to_all, op="sum", async_op=True, pipeline=pipe)
        for t in tensors] and pipe.flush())
    # buckets 1 and 3 share a launch with the reduce of the bucket before; bucket 2 (33,333 elements: chunks that are
    # not 16-byte aligned) has no shared grid and goes out as separate launches
    assert sum(c for name, c in counts.items() if "bucket_step_kernel" in name) == 2
    with pytest.raises(ValueError, match="async_op=True"):
        compressed_reduce_scatter_shard(tensors[0], config=CFG, world_size=world, rank=0, all_to_all=loopback_all_to_all,
                                        pipeline=pipe)


def test_hook_with_the_pipelined_transport_on_a_stream_of_buckets(hip_device):
    """``create_ddp_comm_hook(strategy="reduce_scatter")`` over the pipelined transport: futures in arrival order, the
    flush after the last bucket, results equal to the hook over the unpipelined transport."""
    world, buckets = 8, 9
    piped, plain = transports(world, error_feedback=True)
    hooks = [create_ddp_comm_hook(CFG, strategy="reduce_scatter", reduce="mean", reduce_scatter_all_gather=t)
             for t in (piped, plain)]
    sizes = [G * world * 64] * (buckets - 1) + [G * world * 20 + 24]
    for step in range(2):
        fresh = [grad(n, torch.bfloat16, 500 + 20 * step + k, hip_device) for k, n in enumerate(sizes)]
        if step == 0:
            mine, theirs = [t.clone() for t in fresh], [t.clone() for t in fresh]
        else:
            for k, t in enumerate(fresh):
                mine[k].copy_(t)
                theirs[k].copy_(t)
        futures = [hooks[0](None, Bucket(t, k, last=(k == buckets - 1))) for k, t in enumerate(mine)]
        assert all(f.done() for f in futures)                 # the hook flushed after the last bucket
        wanted = [hooks[1](None, Bucket(t, k, last=(k == buckets - 1))).wait() for k, t in enumerate(theirs)]
        torch.cuda.synchronize()
        for k, (future, want) in enumerate(zip(futures, wanted)):
            assert same_bits(future.wait(), want), f"bucket {k}, step {step}"
    assert piped.pipeline.stats["flushes"] == 2


@pytest.mark.parametrize("error_feedback", [False, True])
@pytest.mark.parametrize("lanes", [1, 2])
def test_an_iteration_of_the_pipeline_captured_in_a_hip_graph_replays_like_eager(hip_device, error_feedback, lanes):
    """No entry point allocates, clears memory or synchronises, so one iteration of the pipelined stream - every
    bucket's launch, the exchanges, the flush, with two lanes the forks and joins of their streams - can be captured
    once and replayed.  Every replay, with the program's own eager work and synchronisations in between, must leave what
    an eager iteration leaves from the same state."""
    world, count = 8, 6
    sizes = [G * world * 48] * 4 + [G * world * 20, G * world * 48]
    piped, _plain = transports(world, error_feedback=error_feedback, lanes=lanes)
    source = [grad(n, torch.bfloat16, 9100 + k, hip_device) for k, n in enumerate(sizes)]
    buckets = [s.clone() for s in source]

    def restore():
        for bucket, s in zip(buckets, source):
            bucket.copy_(s)
        for residual in piped.residuals.values():
            residual.zero_()

    def iteration():
        for bucket in buckets:
            piped(bucket, config=CFG, op="mean")
        piped.flush()

    for _ in range(2):                    # plans, bound launches, residuals and lane streams exist before the capture
        iteration()
    restore()
    iteration()
    torch.cuda.synchronize()
    want = [bucket.clone() for bucket in buckets]
    want_residuals = [r.clone() for r in piped.residuals.values()]
    assert len(want_residuals) == (count if error_feedback else 0)
    restore()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        iteration()
    for replay in range(4):
        restore()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k, (bucket, expected) in enumerate(zip(buckets, want)):
            assert same_bits(bucket, expected), f"bucket {k}, replay {replay}"
        for k, (residual, expected) in enumerate(zip(piped.residuals.values(), want_residuals)):
            assert same_bits(residual, expected), f"residual {k}, replay {replay}"
        # eager work of the same program between the replays: an iteration outside the graph, and a host read-back
        restore()
        iteration()
        assert same_bits(buckets[0], want[0])
