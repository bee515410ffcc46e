"""GPU parity at the full sizes of the benchmark configurations, against the CPU oracle.

The parametrised parity tests cover every type, group size, alignment and payload count on small tensors; these
run the large workloads once, at their real sizes, with the library's own access rule:

  config 2'  the W=8 fused reduce of a whole 100 MiB fp32 bucket (26,214,400 elements), three windows
  config 3   error-feedback quantize of a 100 MiB bf16 bucket (52,428,800 values) with an fp32 residual, 10 steps
  config 4   the reduce-scatter + all-gather plan of a 200 MiB fp32 bucket at W=8, three of the eight shards
  config 5   the Llama-3-8B-shaped bf16 gradient stream in 25 MiB buckets through the workspace pool

Bar: codes, scales, packed bytes, reduced values and residuals bit-exact.
"""
import numpy as np
import pytest
import torch

from oracle import codec_torch

pytestmark = pytest.mark.gpu

G = 64
SEED = 1234


def gen(seed, numel, sigma, device, dtype=torch.float32):
    g = torch.Generator(device=device).manual_seed(seed)
    return (torch.randn(numel, generator=g, device=device) * sigma).to(dtype)


def same_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    if a.dtype != b.dtype or a.shape != b.shape:
        return False
    view = torch.int32 if a.dtype == torch.float32 else torch.int16
    return torch.equal(a.view(view), b.view(view))


@pytest.fixture(scope="module")
def ops(hip_device):
    from lowbit_comm_amd.hip import ops as hip_ops

    return hip_ops


def test_config3_error_feedback_quantize_of_a_100_mib_bf16_bucket_ten_steps(ops, hip_device):
    n, steps = 52_428_800, 10
    groups = ops.num_groups(n, G)
    residual = gen(SEED + 3, n, 1e-5, hip_device)
    cpu_residual = residual.cpu()
    codes = torch.empty(groups * G, dtype=torch.int8, device=hip_device)
    scales = torch.empty(groups, device=hip_device)
    for step in range(steps):
        grad = gen(SEED + 4 + step, n, 1e-3, hip_device, torch.bfloat16)
        assert ops.quant_pack_into(grad, codes, scales, residual=residual, new_residual=residual)
        w_codes, w_scales, _restored, cpu_residual = codec_torch.ef_round_trip(grad.cpu(), cpu_residual, G, "fp32")
        assert torch.equal(codes.cpu(), w_codes), f"codes, step {step}"
        assert same_bits(scales, w_scales), f"scales, step {step}"
        assert same_bits(residual, cpu_residual), f"residual, step {step}"


def test_config2_fused_reduce_of_a_whole_100_mib_bucket_on_three_windows(ops, hip_device):
    n, world, window = 26_214_400, 8, 64 * 16_384
    payloads = [ops.quant_pack(gen(SEED + 20 + r, n, 1e-3, hip_device)) for r in range(world)]
    out = torch.empty(n, device=hip_device)
    assert ops.dequant_reduce_into(payloads, out, divisor=float(world))
    for start in (0, (n // 2) // G * G, n - window):
        peers = [(c[start:start + window].cpu(), s[start // G:(start + window) // G].cpu()) for c, s in payloads]
        want = codec_torch.reduce_payloads(peers, window, G, "fp32", "mean")
        assert same_bits(out[start:start + window], want), f"window at {start}"
    # the other elements: the fused launch against the same reduce done shard by shard (shard-sized launches take
    # another cache policy and block order)
    shard = n // world
    piece = torch.empty(shard, device=hip_device)
    for d in range(world):
        rows = [(c[d * shard:(d + 1) * shard], s[d * shard // G:(d + 1) * shard // G]) for c, s in payloads]
        assert ops.dequant_reduce_into(rows, piece, divisor=float(world))
        assert torch.equal(out[d * shard:(d + 1) * shard].view(torch.int32), piece.view(torch.int32)), f"shard {d}"


def test_config4_reduce_scatter_all_gather_plan_of_a_200_mib_bucket(ops, hip_device):
    from lowbit_comm_amd import CompressionConfig
    from lowbit_comm_amd.hip.reduce_scatter import ReduceScatterPlan

    n, world = 52_428_800, 8
    shard = n // world
    cfg = CompressionConfig(bit=8, group_size=G)
    peers = [gen(SEED + 40 + r, n, 1e-3, hip_device) for r in range(world)]
    plans = [ReduceScatterPlan(n, torch.float32, world_size=world, rank=r, config=cfg, device=hip_device)
             for r in range(world)]
    for plan, bucket in zip(plans, peers):
        plan.quantize_chunks(bucket)
    for r, plan in enumerate(plans):                     # the all-to-all, done by copies
        for src in range(world):
            plan.received[src].copy_(plans[src].send[r])
        plan.reduce_received(op="sum")
        plan.requantize_shard()
    for plan in plans:                                   # the all-gather
        for src in range(world):
            plan.gathered[src].copy_(plans[src].gathered[src])
    out = torch.empty(n, device=hip_device)
    plans[0].decode_gathered(out=out)
    nbytes = plans[0].payload_bytes
    for d in (0, 3, 7):                                  # three of the eight shards through all four stages
        sent = [codec_torch.quantize(p[d * shard:(d + 1) * shard].cpu(), G) for p in peers]
        for src in (0, 5):
            assert torch.equal(plans[src].send[d, :nbytes].cpu(), codec_torch.pack(*sent[src])), f"chunk {d} of rank {src}"
        reduced = codec_torch.reduce_payloads(sent, shard, G, "fp32", "sum")
        assert same_bits(plans[d].shard, reduced), f"reduced shard {d}"
        again = codec_torch.quantize(reduced, G)
        assert torch.equal(plans[0].gathered[d, :nbytes].cpu(), codec_torch.pack(*again)), f"requantized shard {d}"
        assert same_bits(out[d * shard:(d + 1) * shard], codec_torch.dequantize(*again, shard, G, "fp32")), f"decoded shard {d}"
        # the fused reduce + requantize writes the same payload without the fp32 shard
        plans[d].gathered[d].zero_()
        assert torch.equal(plans[d].reduce_and_requantize(op="sum")[:nbytes].cpu(), codec_torch.pack(*again)), f"fused {d}"
    # every other element of the result: decoding is the same launch for all shards, so idempotence covers them
    requantized = [ops.quant_pack(out[d * shard:(d + 1) * shard]) for d in range(world)]
    for d in range(world):
        assert torch.equal(ops.dequant(*requantized[d], shard).view(torch.int32),
                           out[d * shard:(d + 1) * shard].view(torch.int32)), f"idempotence, shard {d}"


def test_config5_llama_3_8b_shaped_stream_through_the_workspace_pool(ops, hip_device):
    from lowbit_comm_amd import CompressionConfig
    from lowbit_comm_amd.hip import ShardWorkspaceProvider, StreamOrderedCompletion, WorkspaceKey, create_torch_workspace_pool

    dev = hip_device
    cfg = CompressionConfig(bit=8, group_size=G)
    hidden, ffn, kv_dim, vocab, layers, world = 4096, 14336, 1024, 128256, 32, 8
    shapes = [(vocab, hidden)]
    for _ in range(layers):
        shapes += [(hidden, hidden), (kv_dim, hidden), (kv_dim, hidden), (hidden, hidden), (ffn, hidden), (ffn, hidden),
                   (hidden, ffn), (hidden,), (hidden,)]
    shapes += [(hidden,), (vocab, hidden)]
    total = sum(int(np.prod(s)) for s in shapes)
    assert total == 8_030_261_248
    bucket_numel = 13_107_200                            # 25 MiB of bf16
    bounds = [(a, min(a + bucket_numel, total)) for a in range(0, total, bucket_numel)]
    assert len(bounds) == 613 and bounds[-1][1] - bounds[-1][0] == 8_654_848
    grads = torch.empty(total, dtype=torch.bfloat16, device=dev)
    residuals = torch.empty(total, dtype=torch.float32, device=dev)
    for index, (a, b) in enumerate(bounds):              # the flattened stream is i.i.d.: generated bucket by bucket
        grads[a:b] = gen(SEED + 5 + index, b - a, 1e-3, dev, torch.bfloat16)
        residuals[a:b] = gen(SEED + 50_000 + index, b - a, 1e-5, dev)
    pool = create_torch_workspace_pool()
    provider = ShardWorkspaceProvider(pool, backend="hip", collective="reduce_scatter", strategy="compressed",
                                      device=str(dev))
    stream = torch.cuda.current_stream(dev)
    peer_rows = {}

    def peers_for(size, index):
        shard = -(-size // world)
        sets = peer_rows.setdefault(size, [])
        want = 4 if size == bucket_numel else 1
        while len(sets) < want:
            rows = torch.empty(world, ops.payload_nbytes(shard, G), dtype=torch.uint8, device=dev)
            for r in range(world):
                assert ops.quant_pack_payload_into(gen(SEED + 90_000 + 8 * len(sets) + r, shard, 1e-3, dev), rows[r])
            sets.append([ops.split_payload(rows[r], shard, G) for r in range(world)])
        return sets[index % len(sets)]

    send_keys = {}

    def send_matrix(session, size, shard):
        key = send_keys.get(size)
        if key is None:
            stride = -(-ops.payload_nbytes(shard, G) // 256) * 256
            key = send_keys[size] = WorkspaceKey(
                backend="hip", collective="reduce_scatter", strategy="compressed", shape_class=(world, stride),
                dtype="uint8", world_size=world, bit=8, group_size=G, chunk_config=(size,), workspace_kind="send",
                device=str(dev))
        return session.acquire(key)

    bound = {}

    def one_pass(check=()):
        seen = {}
        for index, (a, b) in enumerate(bounds):
            size = b - a
            shard = -(-size // world)
            session = provider.begin(stream=stream)
            rows = send_matrix(session, size, shard)
            out = session.get_reduced_shard(index, residuals[:0], (shard,), cfg, dtype="fp32", world_size=world, rank=0)
            entry = bound.get(index)
            if entry is None or entry[2] != (rows.data_ptr(), out.data_ptr()):
                peers = peers_for(size, index)
                entry = bound[index] = (
                    ops.bind_quant_pack_chunks(grads[a:b], rows, world, residual=residuals[a:b], new_residual=residuals[a:b]),
                    ops.bind_dequant_reduce(peers, out, numel=shard), (rows.data_ptr(), out.data_ptr()), peers)
            if index in check:
                seen[index] = (grads[a:b].cpu(), residuals[a:b].cpu())
            entry[0]()
            entry[1]()
            if index in check:
                torch.cuda.synchronize()
                seen[index] += (rows.cpu(), residuals[a:b].cpu(), out[:shard].cpu(), entry[3])
            session.release(completion=StreamOrderedCompletion(stream))
        return seen

    first = one_pass(check=(0, 306, 612))
    torch.cuda.synchronize()
    for index, (g_cpu, r_cpu, rows_cpu, new_r, reduced, peers) in first.items():
        size = g_cpu.numel()
        shard = -(-size // world)
        prepared = torch.cat([g_cpu.float() + r_cpu, torch.zeros(shard * world - size)])
        want_r = torch.empty(shard * world)
        for d in range(world):
            chunk = prepared[d * shard:(d + 1) * shard]
            codes, scales = codec_torch.quantize(chunk, G)
            assert torch.equal(rows_cpu[d, :ops.payload_nbytes(shard, G)], codec_torch.pack(codes, scales)), (index, d)
            want_r[d * shard:(d + 1) * shard] = chunk - codec_torch.dequantize(codes, scales, shard, G, "fp32")
        assert same_bits(new_r, want_r[:size]), f"residual of bucket {index}"
        want = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in peers], shard, G, "fp32", "sum")
        assert same_bits(reduced, want), f"reduced shard of bucket {index}"
    # the pool: one miss per distinct workspace key (send matrix and reduced shard, for the full and the tail size),
    # and nothing allocated by the second pass
    misses = pool.stats.misses
    assert misses == 4
    allocated = torch.cuda.memory_allocated()
    one_pass()
    torch.cuda.synchronize()
    assert pool.stats.misses == misses
    assert torch.cuda.memory_allocated() == allocated

    # the same stream as a pipeline, one launch per bucket: the quantize of bucket k shares its grid with the reduce
    # of what arrived for bucket k-1.  From the same residual state it must leave the same residuals and shards.
    def shared_pass(keep=()):
        kept, previous = {}, None
        for index, (a, b) in enumerate(bounds):
            session = provider.begin(stream=stream)
            size = b - a
            shard = -(-size // world)
            rows = send_matrix(session, size, shard)
            out = session.get_reduced_shard(index, residuals[:0], (shard,), cfg, dtype="fp32", world_size=world, rank=0)
            entry = bound[index]
            assert entry[2] == (rows.data_ptr(), out.data_ptr())
            if previous is None:
                entry[0]()
            else:
                assert ops.bind_quant_chunks_and_reduce(entry[0], previous[1][1])() is True
                if previous[0] in keep:
                    kept[previous[0]] = previous[3][:previous[2]].clone()
            previous = (index, entry, shard, out)          # the shard buffer this bucket's reduce is bound to
            session.release(completion=StreamOrderedCompletion(stream))
        previous[1][1]()
        if previous[0] in keep:
            kept[previous[0]] = previous[3][:previous[2]].clone()
        return kept

    sample = (0, 306, 611, 612)
    start_state = residuals.clone()
    one_pass()
    want_residuals = residuals.clone()
    want_shards = {}
    for index in sample:                                 # the two-launch schedule overwrites the pooled shard: redo these
        size = bounds[index][1] - bounds[index][0]
        shard = -(-size // world)
        piece = torch.empty(shard, device=dev)
        assert ops.dequant_reduce_into(bound[index][3], piece)
        want_shards[index] = piece
    residuals.copy_(start_state)
    got_shards = shared_pass(keep=sample)
    torch.cuda.synchronize()
    assert torch.equal(residuals.view(torch.int32), want_residuals.view(torch.int32))
    for index in sample:
        assert torch.equal(got_shards[index].view(torch.int32), want_shards[index].view(torch.int32)), f"shard of bucket {index}"
    assert pool.stats.misses == misses


def test_config5_stream_through_the_comm_hook_over_the_pipelined_transport(ops, hip_device):
    """The 613-bucket Llama-3-8B-shaped bf16 stream through ``create_ddp_comm_hook(strategy="reduce_scatter")`` over the
    pipelined reduce-scatter transport with local error feedback, W=8, two iterations: every bucket and every residual
    bit-identical to the hook over the unpipelined transport, buckets 0 / 306 / 612 bit-identical to the CPU oracle,
    and one launch per bucket on the device (612 shared launches while the stream arrives + 1 at the flush).  The
    exchanges are stand-ins on the one GPU (this rank's own chunk payloads come back from the all-to-all, its own
    requantized shard fills every row of the all-gather)."""
    from torch.profiler import ProfilerActivity, profile

    from lowbit_comm_amd import CompressionConfig
    from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
    from lowbit_comm_amd.hip.reduce_scatter import make_reduce_scatter_transport

    dev, world = hip_device, 8
    total, bucket_numel = 8_030_261_248, 13_107_200
    bounds = [(a, min(a + bucket_numel, total)) for a in range(0, total, bucket_numel)]
    assert len(bounds) == 613
    sample = (0, 306, 612)

    class Bucket:
        def __init__(self, tensor, index):
            self._tensor, self._index = tensor, index

        def buffer(self):
            return self._tensor

        def index(self):
            return self._index

        def is_last(self):
            return self._index == len(bounds) - 1

    def all_to_all(received, send):
        received.copy_(send)

    def all_gather(gathered, mine):
        gathered[1:, :mine.numel()] = mine

    common = dict(world_size=world, rank=0, all_to_all=all_to_all, all_gather=all_gather, error_feedback=True)
    piped = make_reduce_scatter_transport(pipelined=True, **common)
    plain = make_reduce_scatter_transport(**common)
    cfg = CompressionConfig(bit=8, group_size=G)
    hooks = [create_ddp_comm_hook(cfg, strategy="reduce_scatter", reduce="mean", reduce_scatter_all_gather=t)
             for t in (piped, plain)]
    mine = torch.empty(total, dtype=torch.bfloat16, device=dev)
    theirs = torch.empty(total, dtype=torch.bfloat16, device=dev)
    cpu_residual = {index: None for index in sample}
    for step in range(2):
        inputs = {}
        for index, (a, b) in enumerate(bounds):
            mine[a:b] = gen(SEED + 5 + index + 10_000 * step, b - a, 1e-3, dev, torch.bfloat16)
            if index in sample:
                inputs[index] = mine[a:b].cpu()
        theirs.copy_(mine)
        torch.cuda.synchronize()
        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            futures = [hooks[0](None, Bucket(mine[a:b], index)) for index, (a, b) in enumerate(bounds)]
            torch.cuda.synchronize()
        assert all(f.done() for f in futures)                              # the hook flushed after bucket 612
        names = [e.name for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA and "lbc" in e.name]
        assert sum("bucket_pipeline_step_kernel" in name for name in names) == 613
        assert len(names) == 615                                           # + the first quantize and the last decode
        for index, (a, b) in enumerate(bounds):
            assert futures[index].wait().data_ptr() == mine[a:b].data_ptr()
            hooks[1](None, Bucket(theirs[a:b], index)).wait()
        torch.cuda.synchronize()
        assert torch.equal(mine.view(torch.int16), theirs.view(torch.int16)), f"reduced buckets, iteration {step}"
        for index, (a, b) in enumerate(bounds):
            got = piped.residuals[(mine[a:b].data_ptr(), b - a, torch.bfloat16)]
            want = plain.residuals[(theirs[a:b].data_ptr(), b - a, torch.bfloat16)]
            assert torch.equal(got.view(torch.int32), want.view(torch.int32)), f"residual of bucket {index}, iteration {step}"
        for index in sample:
            a, b = bounds[index]
            size = b - a
            shard = -(-size // world)
            prepared = inputs[index] if cpu_residual[index] is None else inputs[index] + cpu_residual[index]
            padded = torch.cat([prepared, prepared.new_zeros(shard * world - size)])
            payloads, dropped = [], []
            for d in range(world):
                chunk = padded[d * shard:(d + 1) * shard]
                codes, scales = codec_torch.quantize(chunk, G)
                payloads.append((codes, scales))
                dropped.append(chunk - codec_torch.dequantize(codes, scales, shard, G, "fp32"))
            reduced = codec_torch.reduce_payloads(payloads, shard, G, "bf16", "mean")
            again = codec_torch.dequantize(*codec_torch.quantize(reduced, G), shard, G, "bf16")
            assert same_bits(mine[a:b], again.repeat(world)[:size]), f"bucket {index}, iteration {step}, against the oracle"
            cpu_residual[index] = torch.cat(dropped)[:size]
            got = piped.residuals[(mine[a:b].data_ptr(), size, torch.bfloat16)]
            assert same_bits(got, cpu_residual[index]), f"residual of bucket {index}, iteration {step}, against the oracle"
    stats = piped.pipeline.stats
    assert stats["buckets"] == 2 * 613 and stats["merged_launches"] == 2 * 613 and stats["separate_launches"] == 4
