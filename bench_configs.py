#!/usr/bin/env python3
"""Per-configuration measurements of the compression hot path on one MI355X.

Runs the five workloads the headline metric is defined over (synthetic data, one GPU, peers
synthesised in HBM), checks each against the CPU oracle where the size allows, and prints one JSON
object per configuration plus a summary table on stderr:

  1  25 MiB fp32 DDP bucket with 0.1 % outliers: quantize+pack, dequantize, round trip
  2  W=8 fused dequant-reduce of one rank's shard of a 100 MiB fp32 bucket (and the full-bucket shape)
  3  error-feedback quantize of a 100 MiB bf16 bucket with an fp32 residual, 10 steps
  4  full compressed reduce-scatter + all-gather plan of a 200 MiB fp32 bucket at W=8
  5  Llama-3-8B-shaped bf16 gradient stream in 25 MiB buckets: EF quant-pack + W=8 shard reduce per
     bucket through the workspace pool
  6  the same bucket shapes in the byte format of the reference's CUDA extension (scales in the tensor
     dtype, interleaved or appended): quantize+pack, W=8 fused reduce, mean + error-feedback reduce
  7  the host side: the DDP communication hook per bucket (all_gather strategy through the codec facade; reduce-scatter
     strategy over pre-bound plans, without and with error feedback), a pre-bound launch, and the config-5 launch
     sequence eager against one HIP-graph replay.  Rows report host microseconds per bucket next to wall time.

  8  the compute steps of the quantized ring all-reduce on one chunk (an eighth of the config-4 and config-5
     buckets): the fused ring step (decode + accumulate [+ mean] + requantize in one launch) against the separate
     decode-accumulate and quantize launches, and one rank's whole W=8 schedule through the executor

"~N(0, s)" is read as standard deviation s.  Times are HIP-event averages over back-to-back launches that rotate over buffer sets larger than the
last-level cache: "us" is the median of five such batches, "us_min" the fastest batch.

    python bench_configs.py [--configs 1,2,3,4,5,6,7,8] [--no-parity] [--llama-layers 32]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12
SEED = 1234
G = 64


MANIFEST = os.path.join(ROOT, "profiles", "baseline_manifest.json")


GATE_ROWS = ("quant_pack_chunks_100MiB_fp32_W8", "dequant_reduce_shard_3276800_W8", "dequant_reduce_full_26214400_W8",
             "ef_quant_pack_100MiB_bf16_fp32_residual", "bucket_step_25MiB_bf16_ef_plus_shard_reduce_W8",
             "pipeline_step_25MiB_bf16_ef_W8")
GATE_ROW_NAMES = frozenset(GATE_ROWS)


def gate_rows(quads: int = 3, only=None):
    """The six hot-path launches a later change is held to, each timed against a plain 100 MiB device copy in
    A-B-B-A order (copy, kernel, kernel, copy; the reference's gate alternates baseline and candidate the same way,
    tests/benchmarks/fused_dequant_executor_gate.py:16-33) so that clock and thermal drift cancel in the ratio.
    Returns ``{name: {"us", "copy_us", "ratio", "algorithmic_bytes", "frac_of_hbm_peak"}}``; ``ratio`` is the smallest
    kernel/copy ratio over ``quads`` A-B-B-A rounds.  Buffers rotate through more than 600 MB per row.  ``only``: a
    collection of row names to measure instead of all six."""
    import torch

    from lowbit_comm_amd.hip import ops

    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream(dev)

    def gen(seed, numel, sigma, dtype=torch.float32):
        g = torch.Generator(device=dev).manual_seed(seed)
        return (torch.randn(numel, generator=g, device=dev) * sigma).to(dtype)

    def batch(launches, repeats):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(repeats):
            for launch in launches:
                launch()
        stop.record(stream)
        stop.synchronize()
        return start.elapsed_time(stop) * 1e3 / (repeats * len(launches))          # us per launch

    copy_numel = 26_214_400
    sources = [gen(900 + i, copy_numel, 1.0) for i in range(4)]
    sinks = [torch.empty(copy_numel, device=dev) for _ in range(4)]
    copies = [lambda a=a, b=b: b.copy_(a) for a, b in zip(sources, sinks)]

    def payload_rows(shard, world, seed):
        rows = torch.empty(world, ops.payload_nbytes(shard, G), dtype=torch.uint8, device=dev)
        for r in range(world):
            assert ops.quant_pack_payload_into(gen(seed + r, shard, 1e-3), rows[r])
        return rows

    def build(name):
        world = 8
        if name == "quant_pack_chunks_100MiB_fp32_W8":
            n, shard = 26_214_400, 3_276_800
            stride = -(-ops.payload_nbytes(shard, G) // 256) * 256
            return [ops.bind_quant_pack_chunks(gen(10 + s, n, 1e-3), torch.empty(world, stride, dtype=torch.uint8, device=dev), world)
                    for s in range(6)], n * 4 + world * ops.payload_nbytes(shard, G)
        if name == "dequant_reduce_shard_3276800_W8":
            shard = 3_276_800
            sets = []
            for s in range(16):
                rows = payload_rows(shard, world, 100 + 8 * s) if s < 4 else sets_rows[s % 4].clone()
                if s < 4:
                    sets_rows.append(rows)
                sets.append(ops.bind_dequant_reduce([rows[r] for r in range(world)], torch.empty(shard, device=dev)))
            return sets, world * ops.payload_nbytes(shard, G) + shard * 4
        if name == "dequant_reduce_full_26214400_W8":
            n = 26_214_400
            sets = []
            for s in range(2):
                rows = payload_rows(n, world, 300 + 8 * s)
                sets.append(ops.bind_dequant_reduce([rows[r] for r in range(world)], torch.empty(n, device=dev)))
            return sets, world * ops.payload_nbytes(n, G) + n * 4
        if name == "ef_quant_pack_100MiB_bf16_fp32_residual":
            n = 52_428_800
            groups = ops.num_groups(n, G)
            sets = []
            for s in range(2):
                residual = gen(500 + s, n, 1e-5)
                sets.append(ops.bind_quant_pack(gen(510 + s, n, 1e-3, torch.bfloat16), torch.empty(groups * G, dtype=torch.int8, device=dev),
                                                torch.empty(groups, device=dev), residual=residual, new_residual=residual))
            return sets, n * 10 + groups * (G + 4)
        if name == "bucket_step_25MiB_bf16_ef_plus_shard_reduce_W8":
            n, shard = 13_107_200, 1_638_400
            stride = -(-ops.payload_nbytes(shard, G) // 256) * 256
            sets = []
            for s in range(5):
                residual = gen(700 + s, n, 1e-5)
                quant = ops.bind_quant_pack_chunks(gen(710 + s, n, 1e-3, torch.bfloat16), torch.empty(world, stride, dtype=torch.uint8, device=dev),
                                                   world, residual=residual, new_residual=residual)
                rows = payload_rows(shard, world, 720 + 8 * s)
                reduce = ops.bind_dequant_reduce([rows[r] for r in range(world)], torch.empty(shard, device=dev))
                both = ops.bind_quant_chunks_and_reduce(quant, reduce)
                assert both() is True
                sets.append(both)
            return sets, n * 10 + 2 * world * ops.payload_nbytes(shard, G) + shard * 4
        if name == "pipeline_step_25MiB_bf16_ef_W8":
            # what the comm hook's reduce_scatter strategy launches per bucket: error-feedback quantize of bucket k,
            # reduce + requantize of bucket k-1's shard, decode of bucket k-2's eight gathered shards, one grid
            n, shard = 13_107_200, 1_638_400
            nbytes = ops.payload_nbytes(shard, G)
            stride = -(-nbytes // 256) * 256
            sets = []
            for s in range(5):
                residual = gen(800 + s, n, 1e-5)
                quant = ops.bind_quant_pack_chunks(gen(810 + s, n, 1e-3, torch.bfloat16), torch.empty(world, stride, dtype=torch.uint8, device=dev),
                                                   world, residual=residual, new_residual=residual)
                received, gathered = payload_rows(shard, world, 820 + 8 * s), payload_rows(shard, world, 860 + 8 * s)
                mine = torch.empty(nbytes, dtype=torch.uint8, device=dev)
                reduce = ops.bind_dequant_reduce_quant([ops.split_payload(received[r], shard, G) for r in range(world)],
                                                       *ops.split_payload(mine, shard, G), shard, divisor=float(world),
                                                       mid_dtype=torch.bfloat16)
                decode = ops.bind_dequant_chunks(gathered, torch.empty(n, dtype=torch.bfloat16, device=dev), shard)
                step = ops.bind_bucket_pipeline_step(quant, reduce, decode)
                assert step() is True
                sets.append(step)
            return sets, n * 10 + world * nbytes + (world + 1) * nbytes + world * nbytes + n * 2
        raise KeyError(name)

    rows = {}
    for name in GATE_ROWS:
        if only is not None and name not in only:
            continue
        sets_rows = []
        launches, nbytes = build(name)
        repeats = max(2, 96 // len(launches))
        batch(launches, 1)
        batch(copies, 2)
        best = None
        for _ in range(quads):
            a1 = batch(copies, 6)
            b1 = batch(launches, repeats)
            b2 = batch(launches, repeats)
            a2 = batch(copies, 6)
            entry = ((b1 + b2) / (a1 + a2), min(b1, b2), (a1 + a2) / 2)
            best = entry if best is None or entry[0] < best[0] else best
        rows[name] = {"us": best[1], "copy_us": best[2], "ratio": best[0], "algorithmic_bytes": nbytes,
                      "frac_of_hbm_peak": nbytes / (best[1] * 1e-6) / HBM_PEAK}
        del launches, sets_rows
        torch.cuda.empty_cache()
    return rows


def write_manifest(path: str = MANIFEST, refreeze: bool = False) -> int:
    """Freeze the gate rows.  Rows the committed manifest already holds keep their frozen figures - a baseline that
    moved with every measurement would hold nothing - and only rows it lacks are measured and added; ``refreeze``
    measures all of them anew."""
    import subprocess

    frozen = {}
    if not refreeze and os.path.exists(MANIFEST):
        with open(MANIFEST) as handle:
            frozen = json.load(handle).get("rows", {})
    rows = dict(frozen)
    measured = gate_rows(quads=5, only=None if not frozen else GATE_ROW_NAMES - set(frozen))
    rows.update(measured)
    try:
        commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    except OSError:
        commit = ""
    record = {
        "what": "frozen performance baseline of the hot-path launches on one MI355X: microseconds per launch and the ratio "
                "to a plain 100 MiB device copy timed in A-B-B-A order in the same run (gate_rows in bench_configs.py)",
        "written_by": "python3 bench_configs.py --write-manifest", "commit": commit or None,
        "copy": "torch copy_ of 26,214,400 fp32 elements (104,857,600 bytes read, as many written), four rotating pairs",
        "regression_budget": 0.05, "rows": rows,
    }
    with open(path, "w") as handle:
        json.dump(record, handle, indent=1)
        handle.write("\n")
    for name, row in rows.items():
        print(f"{name:52s} {row['us']:8.2f} us  {row['frac_of_hbm_peak'] * 100:5.1f} % of 8 TB/s  ratio to copy {row['ratio']:.4f}",
              file=sys.stderr)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--configs", default="1,2,3,4,5,6,7,8")
    ap.add_argument("--no-parity", action="store_true", help="skip the CPU oracle comparisons")
    ap.add_argument("--llama-layers", type=int, default=32, help="config 5: number of transformer layers (32 = full model)")
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--write-manifest", nargs="?", const=MANIFEST, default=None, metavar="PATH",
                    help="measure the gate rows the committed manifest lacks and write it with them added (default: "
                         "profiles/baseline_manifest.json), then exit")
    ap.add_argument("--refreeze", action="store_true", help="with --write-manifest: measure every gate row anew")
    args = ap.parse_args()
    if args.write_manifest:
        return write_manifest(args.write_manifest, refreeze=args.refreeze)
    wanted = {int(c) for c in args.configs.split(",") if c}

    import torch

    from lowbit_comm_amd import CompressionConfig
    from lowbit_comm_amd.hip import ShardWorkspaceProvider, StreamOrderedCompletion, create_torch_workspace_pool, ops
    from lowbit_comm_amd.hip.reduce_scatter import ReduceScatterPlan

    if not torch.cuda.is_available():
        print("bench_configs.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream(dev)
    cfg = CompressionConfig()
    parity = not args.no_parity
    if parity:
        from oracle import codec_torch
    rows_out = []

    def gen(seed, numel, sigma, dtype=torch.float32, outliers=False):
        g = torch.Generator(device=dev).manual_seed(seed)
        x = torch.randn(numel, generator=g, device=dev) * sigma
        if outliers:
            mask = torch.rand(numel, generator=g, device=dev) < 1e-3
            x = torch.where(mask, torch.randn(numel, generator=g, device=dev) * 1e-1, x)
        return x.to(dtype)

    class Seconds(float):
        """Median over the timed batches; ``best`` is the fastest batch."""

        best = None

    def timed(fn, count, warmup=5, batches=5, warm_seconds=0.05):
        # The parity checks in between leave the GPU idle; launches go on until the clocks are back up.
        started, i = time.perf_counter(), 0
        while i < warmup or time.perf_counter() - started < warm_seconds:
            fn(i)
            i += 1
            if i % 16 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        means = []
        for _ in range(batches):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            for i in range(count):
                fn(i)
            b.record(stream)
            torch.cuda.synchronize()
            means.append(a.elapsed_time(b) * 1e-3 / count)
        result = Seconds(sorted(means)[len(means) // 2])
        result.best = min(means)
        return result

    def bits_equal(a, b):
        a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
        if a.dtype != b.dtype or a.shape != b.shape:
            return False
        view = {4: torch.int32, 2: torch.int16, 1: torch.int8}[a.element_size()]
        return bool(torch.equal(a.view(view), b.view(view)))

    def emit(config, op, nbytes, seconds, input_bytes, check=None, **extra):
        row = {"config": config, "op": op, "us": seconds * 1e6, "algorithmic_bytes": nbytes,
               "achieved_GBps": nbytes / seconds / 1e9, "frac_of_hbm_peak": nbytes / seconds / HBM_PEAK,
               "input_GBps": input_bytes / seconds / 1e9, "parity": check}
        if getattr(seconds, "best", None) is not None:
            row["us_min"] = seconds.best * 1e6
        row.update(extra)
        rows_out.append(row)
        print(json.dumps(row), flush=True)

    def cpu_time(fn, repeats=5):
        fn()
        times = []
        for _ in range(repeats):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        return sorted(times)[len(times) // 2]

    # ------------------------------------------------------------------------------------------ 1
    if 1 in wanted:
        n = 6_553_600
        sets = []
        for s in range(8):          # 8 x 33 MB: rotate past the last-level cache
            x = gen(SEED + 1 + 10 * s, n, 1e-3, outliers=True)
            payload = torch.empty(ops.payload_nbytes(n, G), dtype=torch.uint8, device=dev)
            codes, scales = ops.split_payload(payload, n, G)
            out = torch.empty(n, device=dev)
            sets.append((x, payload, ops.bind_quant_pack(x, codes, scales), ops.bind_dequant(codes, scales, out), out,
                         ops.bind_quant_pack(x, codes, scales, restored=out)))
        check = None
        cpu = {}
        if parity:
            x, payload, q, d, out, both = sets[0]
            q(); d()
            w_codes, w_scales = codec_torch.quantize(x.cpu(), G)
            ok = torch.equal(payload.cpu(), codec_torch.pack(w_codes, w_scales))
            ok = ok and bits_equal(out, codec_torch.dequantize(w_codes, w_scales, n, G, "fp32"))
            payload.zero_(); out.zero_()
            both()                                  # the same two results from one launch
            ok = ok and torch.equal(payload.cpu(), codec_torch.pack(w_codes, w_scales))
            ok = ok and bits_equal(out, codec_torch.dequantize(w_codes, w_scales, n, G, "fp32"))
            rel = float((x - out).norm() / x.norm())
            check = "bit-exact" if ok else "MISMATCH"
            x_cpu = x.cpu()
            cpu["cpu_round_trip_ms"] = cpu_time(lambda: codec_torch.dequantize(*codec_torch.quantize(x_cpu, G), n, G)) * 1e3
            cpu["cpu_threads"] = torch.get_num_threads()
            cpu["round_trip_rel_l2"] = rel
        nbytes = n * 4 + ops.payload_nbytes(n, G)
        emit(1, "quantize+pack 25 MiB fp32", nbytes, timed(lambda i: sets[i % 8][2](), args.iters), n * 4, check, **cpu)
        emit(1, "dequantize 25 MiB fp32", nbytes, timed(lambda i: sets[i % 8][3](), args.iters), ops.payload_nbytes(n, G), check)
        emit(1, "round trip (2 launches)", 2 * nbytes, timed(lambda i: (sets[i % 8][2](), sets[i % 8][3]()), args.iters), n * 4, check)
        emit(1, "round trip, one launch (quantize+pack with the decoded tensor as a second output)", nbytes + n * 4,
             timed(lambda i: sets[i % 8][5](), args.iters), n * 4, check)
        emit(1, "quantize+pack 25 MiB fp32, one buffer set (cache-warm, not an HBM figure)", nbytes,
             timed(lambda i: sets[0][2](), args.iters), n * 4, check)
        emit(1, "dequantize 25 MiB fp32, one buffer set (cache-warm, not an HBM figure)", nbytes,
             timed(lambda i: sets[0][3](), args.iters), ops.payload_nbytes(n, G), check)
        del sets

    # ------------------------------------------------------------------------------------------ 2
    if 2 in wanted:
        n, world = 26_214_400, 8
        shard = n // world
        sets = []
        for s in range(8):
            pairs = []
            for r in range(world):
                bucket_slice = gen(SEED + 2 + r + 100 * s, shard, 1e-3)      # rank r's values for shard 0
                pairs.append(ops.quant_pack(bucket_slice, group_size=G))
            out = torch.empty(shard, device=dev)
            sets.append((pairs, out, ops.bind_dequant_reduce(pairs, out)))
        check = None
        cpu = {}
        if parity:
            pairs, out, bound = sets[0]
            bound()
            cpu_pairs = [(c.cpu(), s.cpu()) for c, s in pairs]
            check = "bit-exact" if bits_equal(out, codec_torch.reduce_payloads(cpu_pairs, shard, G, "fp32", "sum")) else "MISMATCH"
            cpu["cpu_reduce_ms"] = cpu_time(lambda: codec_torch.reduce_payloads(cpu_pairs, shard, G, "fp32", "sum")) * 1e3
            cpu["cpu_threads"] = torch.get_num_threads()
        nbytes = world * ops.payload_nbytes(shard, G) + shard * 4
        emit(2, "fused dequant-reduce W=8, one shard", nbytes, timed(lambda i: sets[i % 8][2](), args.iters),
             world * ops.payload_nbytes(shard, G), check, **cpu)
        emit(2, "fused dequant-reduce W=8, one shard, one buffer set (cache-warm, not an HBM figure)", nbytes,
             timed(lambda i: sets[0][2](), args.iters), world * ops.payload_nbytes(shard, G), check)
        del sets
        full = []
        for s in range(2):
            pairs = [ops.quant_pack(gen(SEED + 2000 + r + 10 * s, n, 1e-3), group_size=G) for r in range(world)]
            out = torch.empty(n, device=dev)
            full.append(ops.bind_dequant_reduce(pairs, out))
        nbytes = world * ops.payload_nbytes(n, G) + n * 4
        emit(2, "fused dequant-reduce W=8, full 100 MiB bucket", nbytes, timed(lambda i: full[i % 2](), 20),
             world * ops.payload_nbytes(n, G))
        del full
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------------------------------ 3
    if 3 in wanted:
        n, steps = 52_428_800, 10
        groups = ops.num_groups(n, G)
        for restored_name in ("fp32", "bf16"):
            residual = gen(SEED + 3, n, 1e-5)
            codes = torch.empty(groups * G, dtype=torch.int8, device=dev)
            scales = torch.empty(groups, device=dev)
            grads = [gen(SEED + 3 + 1 + step, n, 1e-3, torch.bfloat16) for step in range(steps)]
            restored = torch.empty(n, dtype=torch.bfloat16, device=dev) if restored_name == "bf16" else None
            bound = [ops.bind_quant_pack(g, codes, scales, residual=residual, new_residual=residual, restored=restored,
                                         restored_dtype=ops.TORCH_DTYPES[restored_name]) for g in grads]
            check = None
            if parity:
                cpu_residual = residual.cpu()
                ok = True
                for step in range(steps):
                    bound[step]()
                    w_codes, w_scales, w_restored, cpu_residual = codec_torch.ef_round_trip(
                        grads[step].cpu(), cpu_residual, G, restored_name)
                    if step in (0, steps - 1):
                        ok = ok and torch.equal(codes.cpu(), w_codes) and bits_equal(scales, w_scales)
                        ok = ok and bits_equal(residual, cpu_residual)
                        if restored is not None:
                            ok = ok and bits_equal(restored, w_restored)
                check = "bit-exact over 10 steps" if ok else "MISMATCH"
            nbytes = n * (2 + 4 + 4) + groups * (G + 4) + (n * 2 if restored is not None else 0)
            seconds = timed(lambda i: bound[i % steps](), steps * 3, warmup=steps)
            emit(3, f"EF quant-pack 100 MiB bf16 + fp32 residual in place (restored {restored_name}"
                    f"{', written' if restored is not None else ''})", nbytes, seconds, n * 2, check, steps=steps)
            del grads, bound, residual, codes, scales, restored
            torch.cuda.empty_cache()

    # ------------------------------------------------------------------------------------------ 4
    if 4 in wanted:
        n, world = 52_428_800, 8
        shard = n // world
        peers = [gen(SEED + 4 + r, n, 1e-3) for r in range(world)]
        plans = [ReduceScatterPlan(n, torch.float32, world_size=world, rank=r, config=cfg, device=dev) for r in range(world)]
        for plan, bucket in zip(plans, peers):
            plan.quantize_chunks(bucket)
        for r, plan in enumerate(plans):
            for src in range(world):
                plan.received[src].copy_(plans[src].send[r])
            plan.reduce_received(op="sum")
            plan.requantize_shard()
        for plan in plans:
            for src in range(world):
                plan.gathered[src].copy_(plans[src].gathered[src])
        out = torch.empty(n, device=dev)
        plans[0].decode_gathered(out=out)
        check = None
        if parity:
            sent = [[codec_torch.quantize(p.cpu()[d * shard:(d + 1) * shard], G) for d in range(world)] for p in peers]
            ok = all(torch.equal(plans[0].send[d, :plans[0].payload_bytes].cpu(), codec_torch.pack(*sent[0][d]))
                     for d in range(world))
            shards = [codec_torch.reduce_payloads([sent[src][d] for src in range(world)], shard, G, "fp32", "sum")
                      for d in range(world)]
            ok = ok and bits_equal(plans[0].shard, shards[0])
            gathered = [codec_torch.quantize(s, G) for s in shards]
            ok = ok and torch.equal(plans[0].gathered[0, :plans[0].payload_bytes].cpu(), codec_torch.pack(*gathered[0]))
            want = torch.cat([codec_torch.dequantize(c, s, shard, G, "fp32") for c, s in gathered])
            ok = ok and bits_equal(out, want)
            check = "bit-exact (all 4 stages)" if ok else "MISMATCH"
            del sent, shards, gathered, want
        plan = plans[0]
        pb = plan.payload_bytes
        b_quant, b_reduce, b_requant, b_decode = n * 4 + world * pb, world * pb + shard * 4, shard * 4 + pb, world * pb + n * 4
        # stage times use launches bound once to the plans' buffers (what the plan caches internally), so the
        # short stages measure the kernels and not the Python bookkeeping of the plan methods
        def stage_launches(p):
            pairs = p._pairs(p.received)
            row = p.payload(p.gathered, p.rank)
            row_codes, row_scales = ops.split_payload(row, shard, G)
            return (ops.bind_dequant_reduce(pairs, p.shard, numel=shard, group_size=G),
                    ops.bind_quant_pack(p.shard, row_codes, row_scales, group_size=G),
                    ops.bind_dequant_reduce_quant(pairs, row_codes, row_scales, shard, group_size=G))

        bound = [stage_launches(p) for p in plans]
        t_quant = timed(lambda i: plans[i % world].quantize_chunks(peers[i % world]), 24)
        t_reduce = timed(lambda i: bound[i % world][0](), 48)
        t_requant = timed(lambda i: bound[i % world][1](), 48)
        outs = [out, torch.empty_like(out)]
        t_decode = timed(lambda i: plans[i % world].decode_gathered(out=outs[i % 2]), 24)

        def whole(i):
            p = plans[i % world]
            p.quantize_chunks(peers[i % world]); p.reduce_received(op="sum"); p.requantize_shard()
            p.decode_gathered(out=outs[i % 2])

        t_plan = timed(whole, 24)
        # variant for callers that only forward the requantized payload: (ii)+(iii) as one launch, the fp32
        # shard is never written
        fused_check = None
        if parity:
            reference_row = plans[0].payload(plans[0].gathered, 0).clone()
            plans[0].gathered[0].zero_()
            fused_row = plans[0].reduce_and_requantize(op="sum")
            fused_check = "bit-exact vs (ii)+(iii)" if torch.equal(fused_row, reference_row) else "MISMATCH"
        t_fused = timed(lambda i: bound[i % world][2](), 48)

        def whole_fused(i):
            p = plans[i % world]
            p.quantize_chunks(peers[i % world]); p.reduce_and_requantize(op="sum")
            p.decode_gathered(out=outs[i % 2])

        t_plan_fused = timed(whole_fused, 24)
        # the same plan on a stream of such buckets: one launch carries the quantize of bucket k, the reduce +
        # requantize of bucket k-1 and the decode of bucket k-2 (lbc_bucket_pipeline_step); the eight plans stand for
        # eight consecutive buckets
        steps = []
        for k in range(world):
            quant = plans[k].bound_quantize(peers[k])
            reduce = plans[k - 1].bound_reduce_requantize(op="sum")
            decode = plans[k - 2].bound_decode(outs[k % 2])
            steps.append(ops.bind_bucket_pipeline_step(quant, reduce, decode))
        pipeline_check = None
        if parity:
            want_row = plans[0].payload(plans[0].gathered, 0).clone()
            want_send = plans[1].send.clone()
            plans[7].decode_gathered(out=outs[0])
            want_out = outs[0].clone()
            plans[0].gathered[0].zero_(); plans[1].send.zero_(); outs[1].zero_()
            ok = steps[1]() is True           # quantize of bucket 1, reduce + requantize of bucket 0, decode of bucket 7
            torch.cuda.synchronize()
            ok = ok and torch.equal(plans[0].payload(plans[0].gathered, 0), want_row) and torch.equal(plans[1].send, want_send)
            ok = ok and bits_equal(outs[1], want_out)
            pipeline_check = "bit-exact vs the three launches" if ok else "MISMATCH"
            del want_row, want_send, want_out

        def pipeline_step(i):
            if not steps[i % world]():
                raise RuntimeError("no shared launch for the three stages")

        t_pipeline = timed(pipeline_step, 24)
        emit(4, "(i) quant-pack 8 chunks of 200 MiB fp32", b_quant, t_quant, n * 4, check)
        emit(4, "(ii) fused dequant-reduce W=8 -> 25 MiB shard", b_reduce, t_reduce, world * pb, check)
        emit(4, "(iii) requantize shard", b_requant, t_requant, shard * 4, check)
        emit(4, "(iv) decode 8 shard payloads -> 200 MiB", b_decode, t_decode, world * pb, check)
        emit(4, "whole plan (4 launches)", b_quant + b_reduce + b_requant + b_decode, t_plan, n * 4, check)
        emit(4, "(ii+iii) fused reduce + requantize, shard not written", world * pb + pb, t_fused, world * pb, fused_check)
        emit(4, "whole plan, fused variant (3 launches)", b_quant + world * pb + pb + b_decode, t_plan_fused, n * 4,
             fused_check)
        emit(4, "whole plan on a stream of buckets, one launch per bucket (quantize of bucket k + reduce and requantize of "
                "bucket k-1 + decode of bucket k-2)", b_quant + world * pb + pb + b_decode, t_pipeline, n * 4, pipeline_check)
        del steps
        del peers, plans, outs, out
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------------------------------ 5
    if 5 in wanted:
        hidden, ffn, kv_dim, vocab, layers, world = 4096, 14336, 1024, 128256, args.llama_layers, 8
        shapes = [(vocab, hidden)]
        for _ in range(layers):
            shapes += [(hidden, hidden), (kv_dim, hidden), (kv_dim, hidden), (hidden, hidden), (ffn, hidden),
                       (ffn, hidden), (hidden, ffn), (hidden,), (hidden,)]
        shapes += [(hidden,), (vocab, hidden)]
        total = 0
        for s in shapes:
            count = 1
            for d in s:
                count *= d
            total += count
        bucket_numel = 13_107_200                      # 25 MiB of bf16
        bounds = [(a, min(a + bucket_numel, total)) for a in range(0, total, bucket_numel)]
        # the flattened reverse-registration-order stream is i.i.d. by construction, so it is generated
        # bucket by bucket directly (same distribution and sizes; tensor boundaries do not affect the kernels)
        grads = torch.empty(total, dtype=torch.bfloat16, device=dev)
        residuals = torch.empty(total, dtype=torch.float32, device=dev)
        for index, (a, b) in enumerate(bounds):
            grads[a:b] = gen(SEED + 5 + index, b - a, 1e-3, torch.bfloat16)
            residuals[a:b] = gen(SEED + 50_000 + index, b - a, 1e-5)
        pool = create_torch_workspace_pool()
        provider = ShardWorkspaceProvider(pool, backend="hip", collective="reduce_scatter", strategy="compressed",
                                          device=str(dev))
        peer_sets = {}                                  # per bucket size: rotating sets of 8 received payload rows

        def peers_for(size):
            if size not in peer_sets:
                shard = -(-size // world)
                sets = []
                for s in range(24 if size == bucket_numel else 1):       # 24 x 13.9 MB > last-level cache
                    rows = torch.empty(world, ops.payload_nbytes(shard, G), dtype=torch.uint8, device=dev)
                    for r in range(world):
                        ops.quant_pack_payload_into(gen(SEED + 90_000 + 8 * s + r, shard, 1e-3), rows[r])
                    sets.append([ops.split_payload(rows[r], shard, G) for r in range(world)])
                peer_sets[size] = sets
            return peer_sets[size]

        from lowbit_comm_amd.hip import WorkspaceKey

        send_keys = {}

        def send_matrix(session, size, shard):
            """One pooled uint8 [W, stride] send matrix per bucket size (all W chunk payloads, one launch)."""
            key = send_keys.get(size)
            if key is None:
                stride = -(-ops.payload_nbytes(shard, G) // 256) * 256
                key = send_keys[size] = WorkspaceKey(
                    backend="hip", collective="reduce_scatter", strategy="compressed", shape_class=(world, stride),
                    dtype="uint8", world_size=world, bit=8, group_size=G, chunk_config=(size,), workspace_kind="send",
                    device=str(dev))
            return session.acquire(key)

        bound_cache = {}
        raw_stream = stream.cuda_stream

        def one_pass(check_indices=()):
            results = {}
            for index, (a, b) in enumerate(bounds):
                size = b - a
                shard = -(-size // world)
                session = provider.begin(stream=stream)
                rows = send_matrix(session, size, shard)
                out = session.get_reduced_shard(index, residuals[:0], (shard,), cfg, dtype="fp32", world_size=world, rank=0)
                cached = bound_cache.get(index)
                if cached is None or cached[2] != (rows.data_ptr(), out.data_ptr()):
                    peers = peers_for(size)[index % len(peers_for(size))]
                    cached = bound_cache[index] = (
                        ops.bind_quant_pack_chunks(grads[a:b], rows, world, residual=residuals[a:b],
                                                   new_residual=residuals[a:b]),
                        ops.bind_dequant_reduce(peers, out, numel=shard), (rows.data_ptr(), out.data_ptr()), peers)
                if index in check_indices:
                    results[index] = (grads[a:b].cpu(), residuals[a:b].cpu())
                cached[0](raw_stream)
                cached[1](raw_stream)
                if index in check_indices:
                    torch.cuda.synchronize()
                    results[index] += (rows.cpu(), residuals[a:b].cpu(), out[:shard].cpu(), cached[3])
                session.release(completion=StreamOrderedCompletion(stream))
            return results

        check = None
        sample = (0, len(bounds) // 2, len(bounds) - 1) if parity else ()
        first = one_pass(sample)
        torch.cuda.synchronize()
        if parity:
            ok = True
            for index, (g_cpu, r_cpu, rows_cpu, new_r, reduced, peers) in first.items():
                size = g_cpu.numel()
                shard = -(-size // world)
                prepared = torch.cat([g_cpu.float() + r_cpu, torch.zeros(shard * world - size)])
                want_r = torch.empty(shard * world)
                for d in range(world):
                    chunk = prepared[d * shard:(d + 1) * shard]
                    codes, scales = codec_torch.quantize(chunk, G)
                    ok = ok and torch.equal(rows_cpu[d, :ops.payload_nbytes(shard, G)], codec_torch.pack(codes, scales))
                    want_r[d * shard:(d + 1) * shard] = chunk - codec_torch.dequantize(codes, scales, shard, G, "fp32")
                ok = ok and bits_equal(new_r, want_r[:size])
                want = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in peers], shard, G, "fp32", "sum")
                ok = ok and bits_equal(reduced, want)
            check = f"bit-exact on buckets {sorted(first)}" if ok else "MISMATCH"
        misses_after_first = pool.stats.misses
        torch.cuda.synchronize()
        allocated = torch.cuda.memory_allocated()
        a_ev, b_ev = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        host0 = time.perf_counter()
        a_ev.record(stream)
        one_pass()
        b_ev.record(stream)
        host1 = time.perf_counter()
        torch.cuda.synchronize()
        seconds = a_ev.elapsed_time(b_ev) * 1e-3
        stats = pool.stats
        nbytes = 0
        for a, b in bounds:
            size = b - a
            shard = -(-size // world)
            pbytes = ops.payload_nbytes(shard, G)
            nbytes += size * (2 + 4 + 4) + world * pbytes + world * pbytes + shard * 4
        emit(5, f"Llama-3-8B-shaped stream ({layers} layers): {len(bounds)} buckets x (EF quant-pack 8 chunks + W=8 shard reduce)",
             nbytes, seconds, total * 2, check, buckets=len(bounds), total_elements=total,
             tail_elements=bounds[-1][1] - bounds[-1][0], us_per_bucket=seconds / len(bounds) * 1e6,
             host_enqueue_s=host1 - host0, pool_misses=stats.misses, pool_misses_after_first_pass=misses_after_first,
             pool_hits=stats.hits, steady_state_allocation_bytes=torch.cuda.memory_allocated() - allocated,
             distinct_workspace_keys=2 * 2)

        # the same stream as a pipeline: the quantize of bucket k shares its grid with the reduce of what arrived for
        # bucket k-1 (one launch per bucket, the last reduce on its own)
        shared = {}

        def one_pass_shared():
            previous = None
            for index, (a, b) in enumerate(bounds):
                size = b - a
                shard = -(-size // world)
                session = provider.begin(stream=stream)
                rows = send_matrix(session, size, shard)
                out = session.get_reduced_shard(index, residuals[:0], (shard,), cfg, dtype="fp32", world_size=world, rank=0)
                cached = bound_cache[index]
                assert cached[2] == (rows.data_ptr(), out.data_ptr())
                if previous is None:
                    cached[0](raw_stream)
                else:
                    both = shared.get(index)
                    if both is None:
                        both = shared[index] = ops.bind_quant_chunks_and_reduce(cached[0], previous[1])
                    if not both(raw_stream):
                        cached[0](raw_stream)
                        previous[1](raw_stream)
                previous = cached
                session.release(completion=StreamOrderedCompletion(stream))
            previous[1](raw_stream)

        shared_check = None
        if parity:
            # both schedules from the same residual state must leave the same residuals and the same last shard
            start_state = residuals.clone()
            one_pass()
            torch.cuda.synchronize()
            want_residuals = residuals.clone()
            last_size = bounds[-1][1] - bounds[-1][0]
            want_last = bound_cache[len(bounds) - 1][1]._keep[1][:-(-last_size // world)].clone()
            residuals.copy_(start_state)
            one_pass_shared()
            torch.cuda.synchronize()
            got_last = bound_cache[len(bounds) - 1][1]._keep[1][:-(-last_size // world)]
            same = torch.equal(residuals.view(torch.int32), want_residuals.view(torch.int32)) and \
                torch.equal(got_last.view(torch.int32), want_last.view(torch.int32))
            shared_check = "bit-exact against the two-launch schedule (all residuals, last shard)" if same else "MISMATCH"
            del start_state, want_residuals
            torch.cuda.empty_cache()
        one_pass_shared()
        torch.cuda.synchronize()
        host0 = time.perf_counter()
        a_ev.record(stream)
        one_pass_shared()
        b_ev.record(stream)
        host1 = time.perf_counter()
        torch.cuda.synchronize()
        seconds = a_ev.elapsed_time(b_ev) * 1e-3
        emit(5, f"same stream, one launch per bucket: EF quant-pack of bucket k + shard reduce of bucket k-1 in one grid",
             nbytes, seconds, total * 2, shared_check, buckets=len(bounds), us_per_bucket=seconds / len(bounds) * 1e6,
             host_enqueue_s=host1 - host0)
        # The same launches dealt to two streams in turn.  Consecutive buckets are independent, so the ramp-up of one
        # bucket's launch overlaps the drain of the one before.  Each stream has its own send matrix and shard output
        # (a bucket's payloads must survive until they are exchanged), hence nothing crosses between the streams.
        from lowbit_comm_amd.hip.lanes import StreamLanes

        lanes = StreamLanes(2, dev)
        lane_buffers = {}
        lane_launches = []

        def lane_buffer(size, shard, lane):
            pair = lane_buffers.get((size, lane))
            if pair is None:
                stride = -(-ops.payload_nbytes(shard, G) // 256) * 256
                pair = lane_buffers[(size, lane)] = (torch.empty(world, stride, dtype=torch.uint8, device=dev),
                                                     torch.empty(shard, device=dev))
            return pair

        previous = None
        for index, (a, b) in enumerate(bounds):
            size = b - a
            shard = -(-size // world)
            rows, out = lane_buffer(size, shard, index & 1)
            peers = peers_for(size)[index % len(peers_for(size))]
            quant = ops.bind_quant_pack_chunks(grads[a:b], rows, world, residual=residuals[a:b], new_residual=residuals[a:b])
            reduce = ops.bind_dequant_reduce(peers, out, numel=shard)
            lane_launches.append(quant if previous is None else ops.bind_quant_chunks_and_reduce(quant, previous))
            previous = reduce
        last_reduce, last_out = previous, out

        def one_pass_two_streams():
            lanes.fork()
            for index, launch in enumerate(lane_launches):
                if not launch(lanes.handle(index)):
                    raise RuntimeError("no shared launch for this bucket")
            last_reduce(lanes.handle(len(lane_launches)))
            lanes.join()

        lanes_check = None
        if parity:
            start_state = residuals.clone()
            one_pass()
            torch.cuda.synchronize()
            want_residuals = residuals.clone()
            last_size = bounds[-1][1] - bounds[-1][0]
            want_last = bound_cache[len(bounds) - 1][1]._keep[1][:-(-last_size // world)].clone()
            residuals.copy_(start_state)
            torch.cuda.synchronize()
            one_pass_two_streams()
            torch.cuda.synchronize()
            same = torch.equal(residuals.view(torch.int32), want_residuals.view(torch.int32)) and \
                torch.equal(last_out[:-(-last_size // world)].view(torch.int32), want_last.view(torch.int32))
            lanes_check = "bit-exact against the two-launch schedule (all residuals, last shard)" if same else "MISMATCH"
            del start_state, want_residuals
            torch.cuda.empty_cache()
        one_pass_two_streams()
        torch.cuda.synchronize()
        host0 = time.perf_counter()
        a_ev.record(stream)
        one_pass_two_streams()
        b_ev.record(stream)
        host1 = time.perf_counter()
        torch.cuda.synchronize()
        seconds = a_ev.elapsed_time(b_ev) * 1e-3
        emit(5, "same stream, one launch per bucket, the buckets dealt to two HIP streams in turn (each with its own send "
                "matrix and shard output)", nbytes, seconds, total * 2, lanes_check, buckets=len(bounds),
             us_per_bucket=seconds / len(bounds) * 1e6, host_enqueue_s=host1 - host0)
        del residuals, lane_launches, lane_buffers
        torch.cuda.empty_cache()
        # The whole reduce-scatter + all-gather plan over the same stream, as the comm hook runs it: through
        # create_ddp_comm_hook(strategy="reduce_scatter") over the transport with local error feedback, unpipelined
        # (three launches per bucket) and pipelined (one launch per bucket: quantize of bucket k, reduce + requantize
        # of bucket k-1, decode of bucket k-2).  The exchanges are stand-ins that fill their rows once; parity of this
        # path at full size is tests/test_full_size_configs.py.
        from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
        from lowbit_comm_amd.hip.reduce_scatter import make_reduce_scatter_transport

        class StreamBucket:
            def __init__(self, tensor, index, last):
                self._tensor, self._index, self._last = tensor, index, last

            def buffer(self):
                return self._tensor

            def index(self):
                return self._index

            def is_last(self):
                return self._last

        class Slot:
            def set_result(self, value):
                self.value = value

        hook_buckets = [StreamBucket(grads[a:b], index, index == len(bounds) - 1) for index, (a, b) in enumerate(bounds)]
        plan_bytes = 0
        for a, b in bounds:
            size = b - a
            payload = ops.payload_nbytes(-(-size // world), G)
            plan_bytes += size * (2 + 4 + 4) + world * payload + (world + 1) * payload + world * payload + size * 2
        for pipelined in (False, True):
            filled = set()

            def all_to_all(received, send):
                if received.data_ptr() not in filled:
                    received.copy_(send)
                    filled.add(received.data_ptr())

            def all_gather(gathered, mine):
                if gathered.data_ptr() not in filled:
                    gathered[1:, :mine.numel()] = mine
                    filled.add(gathered.data_ptr())

            transport = make_reduce_scatter_transport(world_size=world, rank=0, all_to_all=all_to_all, all_gather=all_gather,
                                                      error_feedback=True, pipelined=pipelined, future_factory=Slot)
            hook = create_ddp_comm_hook(CompressionConfig(), strategy="reduce_scatter", reduce="mean",
                                        reduce_scatter_all_gather=transport, future_factory=Slot)

            def hook_pass():
                for bucket in hook_buckets:
                    hook(None, bucket)

            hook_pass()
            hook_pass()
            torch.cuda.synchronize()
            host0 = time.perf_counter()
            a_ev.record(stream)
            hook_pass()
            b_ev.record(stream)
            host1 = time.perf_counter()
            torch.cuda.synchronize()
            seconds = a_ev.elapsed_time(b_ev) * 1e-3
            emit(5, "same stream through the comm hook, reduce_scatter strategy, whole plan with error feedback (quantize, "
                    "reduce + requantize, decode of 8 shards per bucket), " +
                    ("pipelined transport: one launch per bucket" if pipelined else "unpipelined transport: three launches per bucket"),
                 plan_bytes, seconds, total * 2, None, buckets=len(bounds), us_per_bucket=seconds / len(bounds) * 1e6,
                 host_enqueue_s=host1 - host0)
            transport.reset()
            del transport, hook
            torch.cuda.empty_cache()
        del grads, hook_buckets
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------------------------------ 6
    if 6 in wanted:
        from lowbit_comm_amd.hip import cuda_wire

        if parity:
            from oracle import cuda_wire_scalar as wire_c

        def host(t):
            t = t.detach().cpu().contiguous()
            return t.view(torch.int16).numpy().view("uint16") if t.dtype == torch.bfloat16 else t.numpy()

        # The one kernel-level figure the reference publishes (an RTX A6000): its fused input + residual -> quantize+pack
        # on 8,388,608 fp16 elements, group 64, 0.17072 ms.  Same shape here, in its byte format and in the portable one.
        m = 8_388_608
        published_ms = 0.17072
        sets_n = 12                       # 12 x 42 MB: rotate past the last-level cache
        gs = [gen(SEED + 1200 + s, m, 1e-3, torch.float16) for s in range(sets_n)]
        rs = [gen(SEED + 1300 + s, m, 1e-5, torch.float16) for s in range(sets_n)]
        pb = cuda_wire.payload_nbytes(m, torch.float16)
        outs = [torch.empty(pb, dtype=torch.uint8, device=dev) for _ in range(sets_n)]
        wire = [cuda_wire.bind_quant_pack(gs[s], outs[s], residual=rs[s]) for s in range(sets_n)]
        check = None
        if parity:
            wire[0]()
            want = wire_c.quantize(host(gs[0]), "fp16", 64, True, residual=host(rs[0]))
            check = "bit-exact" if host(outs[0]).tobytes() == want.tobytes() else "MISMATCH"
        seconds = timed(lambda i: wire[i % sets_n](), args.iters * 4)
        emit(6, f"input + residual -> quantize+pack, 8,388,608 fp16, interleaved scales (the reference publishes "
                f"{published_ms} ms for this on an RTX A6000: {published_ms * 1e-3 / seconds:.1f}x)", 2 * m * 2 + pb, seconds,
             m * 2, check, published_ms_rtx_a6000=published_ms)
        port = [torch.empty(ops.payload_nbytes(m, G), dtype=torch.uint8, device=dev) for _ in range(sets_n)]
        portable = [ops.bind_quant_pack(gs[s], *ops.split_payload(port[s], m, G), residual=rs[s]) for s in range(sets_n)]
        check = None
        if parity:
            portable[0]()
            w_codes, w_scales = codec_torch.quantize((gs[0].cpu() + rs[0].cpu()), G)
            check = "bit-exact" if torch.equal(port[0].cpu(), codec_torch.pack(w_codes, w_scales)) else "MISMATCH"
        emit(6, "the same shape in the portable format (fp16 sum, fp32 scales)", 2 * m * 2 + ops.payload_nbytes(m, G),
             timed(lambda i: portable[i % sets_n](), args.iters * 4), m * 2, check)
        del gs, rs, outs, wire, port, portable

        world, n = 8, 26_214_400
        for name, dtype in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
            item = 4 if name == "fp32" else 2
            for compact in (True, False):
                layout = "interleaved scales" if compact else "appended scales"
                pbytes = cuda_wire.payload_nbytes(n, dtype)
                xs = [gen(SEED + 600 + s, n, 1e-3, dtype) for s in range(4)]
                outs = [torch.empty(pbytes, dtype=torch.uint8, device=dev) for _ in range(4)]
                quant = [cuda_wire.bind_quant_pack(xs[s], outs[s], compact=compact) for s in range(4)]
                check = None
                if parity:
                    quant[0]()
                    check = "bit-exact" if host(outs[0]).tobytes() == wire_c.quantize(host(xs[0]), name, 64, compact).tobytes() else "MISMATCH"
                emit(6, f"quantize+pack 26.2M {name}, {layout}", n * item + pbytes,
                     timed(lambda i: quant[i % 4](), args.iters), n * item, check)
                # W=8 fused reduce (+ mean + error feedback) of full-bucket payloads; parity on one shard-sized case
                payloads = [[cuda_wire.quant_pack(gen(SEED + 700 + 10 * s + r, n, 1e-3, dtype), compact=compact)
                             for r in range(world)] for s in range(2)]
                res = [torch.empty(n, dtype=dtype, device=dev) for _ in range(2)]
                prepared = [gen(SEED + 800 + s, n, 1e-3, dtype) for s in range(2)]
                plain = [cuda_wire.bind_dequant_reduce(payloads[s], res[s], compact=compact, inv_divisor=0.125) for s in range(2)]
                feedback = [cuda_wire.bind_dequant_reduce(payloads[s], res[s], compact=compact, inv_divisor=0.125,
                                                          prepared=prepared[s], new_residual=prepared[s]) for s in range(2)]
                check = None
                if parity:
                    m = n // world
                    small = [cuda_wire.quant_pack(gen(SEED + 900 + r, m, 1e-3, dtype), compact=compact) for r in range(world)]
                    got = torch.empty(m, dtype=dtype, device=dev)
                    prep = gen(SEED + 950, m, 1e-3, dtype)
                    new_r = torch.empty_like(prep)
                    cuda_wire.dequant_reduce_into(small, got, compact=compact, inv_divisor=0.125, prepared=prep, new_residual=new_r)
                    want, want_r = wire_c.reduce_payloads([host(p) for p in small], m, name, 64, compact, 0.125, True, prepared=host(prep))
                    ok = host(got).tobytes() == want.tobytes() and host(new_r).tobytes() == want_r.tobytes()
                    check = "bit-exact (one shard)" if ok else "MISMATCH"
                emit(6, f"fused dequant-reduce W=8 -> 26.2M {name}, {layout}", world * pbytes + n * item,
                     timed(lambda i: plain[i % 2](), max(10, args.iters // 2)), world * pbytes, check)
                emit(6, f"fused reduce + mean + error feedback W=8, {name}, {layout}", world * pbytes + 3 * n * item,
                     timed(lambda i: feedback[i % 2](), max(10, args.iters // 2)), world * pbytes, check)
                del xs, outs, quant, payloads, res, prepared, plain, feedback
            # 4-bit codes (experimental upstream): quantize+pack and decode of one payload, interleaved scales
            p4 = cuda_wire.payload_nbytes(n, dtype, 64, 4)
            xs = [gen(SEED + 1000 + s, n, 1e-3, dtype) for s in range(4)]
            outs = [torch.empty(p4, dtype=torch.uint8, device=dev) for _ in range(4)]
            back = [torch.empty(n, dtype=dtype, device=dev) for _ in range(4)]
            quant = [cuda_wire.bind_quant_pack(xs[s], outs[s], bit=4) for s in range(4)]
            decode = [cuda_wire.bind_dequant(outs[s], back[s], bit=4) for s in range(4)]
            check = None
            if parity:
                quant[0](); decode[0]()
                want = wire_c.quantize(host(xs[0]), name, 64, True, bit=4)
                ok = host(outs[0]).tobytes() == want.tobytes()
                ok = ok and host(back[0]).tobytes() == wire_c.dequantize(want, n, name, 64, True, bit=4).tobytes()
                check = "bit-exact" if ok else "MISMATCH"
            for s in range(4):
                quant[s]()
            emit(6, f"4-bit quantize+pack 26.2M {name}, interleaved scales", n * item + p4,
                 timed(lambda i: quant[i % 4](), args.iters), n * item, check)
            emit(6, f"4-bit decode 26.2M {name}, interleaved scales", n * item + p4,
                 timed(lambda i: decode[i % 4](), args.iters), p4, check)
            del xs, outs, back, quant, decode
            # the extension's other policies (general kernels): top-k side channel, stochastic rounding, code books
            if parity:
                from oracle import cuda_wire_general_scalar as general_c
            xs = [gen(SEED + 1100 + s, n, 1e-3, dtype) for s in range(4)]
            back = [torch.empty(n, dtype=dtype, device=dev) for _ in range(4)]
            for label, policy, seeds in (
                    ("top-2 outliers, 8-bit linear", dict(bit=8, quant_type="linear", topk=2), None),
                    ("stochastic rounding, 8-bit linear", dict(bit=8, quant_type="linear", topk=0), (SEED, 0)),
                    ("4-bit normal code book", dict(bit=4, quant_type="normal", topk=0), None)):
                pb = cuda_wire.general_payload_nbytes(n, dtype, 64, policy["bit"], policy["topk"])
                outs = [torch.empty(pb, dtype=torch.uint8, device=dev) for _ in range(4)]
                quant = [cuda_wire.bind_quant_general(xs[s], outs[s], compact=True, stochastic=seeds, **policy) for s in range(4)]
                decode = [cuda_wire.bind_dequant_general(outs[s], back[s], compact=True, **policy) for s in range(4)]
                check = None
                if parity:          # the scalar restatement on the first 1 Mi elements (group indices coincide there)
                    m = 1 << 20
                    part = torch.empty(cuda_wire.general_payload_nbytes(m, dtype, 64, policy["bit"], policy["topk"]),
                                       dtype=torch.uint8, device=dev)
                    cuda_wire.quant_general_into(xs[0][:m], part, compact=True, stochastic=seeds, **policy)
                    want = general_c.quantize(host(xs[0][:m]), name, 64, policy["bit"], policy["quant_type"],
                                              policy["topk"], seeds, True)
                    ok = host(part).tobytes() == want.tobytes()
                    got = torch.empty(m, dtype=dtype, device=dev)
                    cuda_wire.dequant_general_into(part, got, compact=True, **policy)
                    ok = ok and host(got).tobytes() == general_c.dequantize(
                        want, m, name, 64, policy["bit"], policy["quant_type"], policy["topk"], True).tobytes()
                    check = "bit-exact (first 1Mi elements)" if ok else "MISMATCH"
                for s in range(4):
                    quant[s]()
                emit(6, f"quantize, {label}, 26.2M {name}", n * item + pb, timed(lambda i: quant[i % 4](), args.iters),
                     n * item, check)
                emit(6, f"decode, {label}, 26.2M {name}", n * item + pb, timed(lambda i: decode[i % 4](), args.iters),
                     pb, check)
                del outs, quant, decode
            del xs, back


    # ------------------------------------------------------------------------------------------ 7
    if 7 in wanted:
        from lowbit_comm_amd.communication import CompressedPayload, GatheredPayloads
        from lowbit_comm_amd.communication.ddp_hook import create_ddp_comm_hook
        from lowbit_comm_amd.hip.loader import load_hip_extension
        from lowbit_comm_amd.hip.reduce_scatter import make_reduce_scatter_transport

        class Bucket:
            def __init__(self, tensor, index):
                self._tensor, self._index = tensor, index

            def buffer(self):
                return self._tensor

            def index(self):
                return self._index

        class Slot:
            def set_result(self, value):
                self.value = value

        def host_and_wall(fn, count):
            for i in range(8):
                fn(i)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(count):
                fn(i)
            host = (time.perf_counter() - t0) / count
            torch.cuda.synchronize()
            return host, (time.perf_counter() - t0) / count

        def host_row(op, host, wall, **extra):
            row = {"config": 7, "op": op, "host_us": host * 1e6, "us": wall * 1e6, "algorithmic_bytes": 0,
                   "achieved_GBps": 0.0, "frac_of_hbm_peak": 0.0, "input_GBps": 0.0, "parity": None}
            row.update(extra)
            rows_out.append(row)
            print(json.dumps(row), flush=True)

        world, n = 8, 13_107_200                                   # a 25 MiB bf16 bucket
        status = load_hip_extension()
        buckets = [Bucket(gen(SEED + 7000 + i, n, 1e-3, torch.bfloat16), i) for i in range(4)]
        # all_gather strategy through the facade: W - 1 stand-in peers resident in HBM
        peers = {}

        def gather(payload):
            key = payload.buffer.numel()
            if key not in peers:       # the peers' payloads stay where they are, as in a reused gather buffer
                peers[key] = [CompressedPayload(buffer=payload.buffer.clone(), shape=payload.shape, dtype=payload.dtype)
                              for _ in range(world - 1)]
            return GatheredPayloads(payloads=[payload] + peers[key], world_size=world)

        for feedback in (False, True):
            hook = create_ddp_comm_hook(CompressionConfig(error_feedback=feedback), strategy="all_gather", reduce="mean",
                                        all_gather=gather, extension_status=status, future_factory=Slot,
                                        workspace_cache_max_entries=8)
            host, wall = host_and_wall(lambda i: hook(None, buckets[i % 4]), 40)
            host_row(f"hook, all_gather strategy through the facade, 25 MiB bf16 bucket, W=8, error feedback {feedback}",
                     host, wall)
        # reduce-scatter strategy over pre-bound plans; the exchanges are stand-ins that fill the rows once
        for feedback in (False, True):
            filled = set()

            def all_to_all(received, send):
                if received.data_ptr() not in filled:
                    for r in range(world):
                        received[r].copy_(send[0])
                    filled.add(received.data_ptr())

            def all_gather(gathered, mine):
                if gathered.data_ptr() not in filled:
                    for r in range(world):
                        gathered[r, :mine.numel()].copy_(mine)
                    filled.add(gathered.data_ptr())

            transport = make_reduce_scatter_transport(world_size=world, rank=0, all_to_all=all_to_all,
                                                      all_gather=all_gather, error_feedback=feedback)
            hook = create_ddp_comm_hook(CompressionConfig(error_feedback=False), strategy="reduce_scatter", reduce="mean",
                                        reduce_scatter_all_gather=transport, future_factory=Slot)
            host, wall = host_and_wall(lambda i: hook(None, buckets[i % 4]), 60)
            host_row(f"hook, reduce_scatter strategy over pre-bound plans, 25 MiB bf16 bucket, W=8, error feedback {feedback}",
                     host, wall)
        # the same strategy over the pipelined transport: one launch per bucket carries the quantize of bucket k, the
        # reduce + requantize of bucket k-1 and the decode of bucket k-2; the hook flushes after the last bucket
        class StreamBucket(Bucket):
            def __init__(self, tensor, index, last):
                super().__init__(tensor, index)
                self._last = last

            def is_last(self):
                return self._last

        stream_count = 16
        stream_buckets = [StreamBucket(gen(SEED + 7500 + i, n, 1e-3, torch.bfloat16), i, i == stream_count - 1)
                          for i in range(stream_count)]
        for feedback in (False, True):
            for lane_count in (1, 2):
                filled = set()
                transport = make_reduce_scatter_transport(world_size=world, rank=0, all_to_all=all_to_all,
                                                          all_gather=all_gather, error_feedback=feedback, pipelined=True,
                                                          lanes=lane_count, future_factory=Slot)
                hook = create_ddp_comm_hook(CompressionConfig(error_feedback=False), strategy="reduce_scatter",
                                            reduce="mean", reduce_scatter_all_gather=transport, future_factory=Slot)

                def one_iteration(_i=0):
                    for bucket in stream_buckets:
                        hook(None, bucket)

                host, wall = host_and_wall(one_iteration, 12)
                stats = transport.pipeline.stats
                host_row(f"hook, reduce_scatter strategy over the pipelined transport ({lane_count} stream"
                         f"{'s' if lane_count > 1 else ''}), stream of {stream_count} 25 MiB bf16 buckets, W=8, error feedback "
                         f"{feedback}, per bucket", host / stream_count, wall / stream_count,
                         merged_launches_per_bucket=stats["merged_launches"] / stats["buckets"],
                         separate_launches_per_bucket=stats["separate_launches"] / stats["buckets"])
                # the same iteration - every bucket through the hook, the exchanges, the flush - as one HIP-graph replay
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    one_iteration()
                host, wall = host_and_wall(lambda i: graph.replay(), 12)
                host_row(f"the same iteration ({lane_count} stream{'s' if lane_count > 1 else ''}, error feedback {feedback}) "
                         "as one HIP-graph replay, per bucket", host / stream_count, wall / stream_count)
                del graph
        # the all-gather form of the all-reduce over pre-bound plans, behind the hook's whole-collective seam: a bucket
        # is quantized into one payload, the W payloads are gathered (W - 1 stand-in peers resident in HBM) and one
        # fused launch reduces them into the bucket.  Sixteen buckets of sixteen sizes, so that every bucket has
        # its own peers' payloads (1.6 GB in all) and no row reads them out of the last-level cache; the facade's own
        # all_gather strategy runs over the same stream for comparison.
        from lowbit_comm_amd.hip.reduce_scatter import make_all_gather_transport

        varied = [StreamBucket(gen(SEED + 7600 + i, n - 64 * world * 8 * i, 1e-3, torch.bfloat16), i, i == stream_count - 1)
                  for i in range(stream_count)]
        whole_filled = set()

        def whole_gather(received, mine):
            if received.data_ptr() not in whole_filled:     # the peers' payloads stay where they are; row 0 is `mine`
                for r in range(1, world):
                    received[r, :mine.numel()].copy_(mine)
                whole_filled.add(received.data_ptr())

        for feedback in (False, True):
            peers.clear()
            hook = create_ddp_comm_hook(CompressionConfig(error_feedback=feedback), strategy="all_gather", reduce="mean",
                                        all_gather=gather, extension_status=status, future_factory=Slot,
                                        workspace_cache_max_entries=2 * stream_count)

            def facade_iteration(_i=0):
                for bucket in varied:
                    hook(None, bucket)

            host, wall = host_and_wall(facade_iteration, 12)
            host_row(f"hook, all_gather strategy through the facade, stream of {stream_count} bf16 buckets of 22-25 MiB with their "
                     f"own peers, W=8, error feedback {feedback}, per bucket", host / stream_count, wall / stream_count)
            for pipelined in (False, True):
                transport = make_all_gather_transport(world_size=world, rank=0, all_gather=whole_gather,
                                                      error_feedback=feedback, pipelined=pipelined, future_factory=Slot)
                hook = create_ddp_comm_hook(CompressionConfig(error_feedback=False), strategy="topology", reduce="mean",
                                            topology_all_reduce=transport, future_factory=Slot)

                def gather_iteration(_i=0):
                    for bucket in varied:
                        hook(None, bucket)

                host, wall = host_and_wall(gather_iteration, 12)
                host_row(f"hook, all-gather form over pre-bound plans ({'pipelined: one launch per bucket' if pipelined else 'two launches per bucket'}), "
                         f"the same stream, W=8, {'local ' if feedback else ''}error feedback {feedback}, per bucket",
                         host / stream_count, wall / stream_count)
                del transport, hook
        peers.clear()
        del varied
        del stream_buckets
        # one pre-bound launch
        x = gen(SEED + 7100, n, 1e-3, torch.bfloat16)
        payload = torch.empty(ops.payload_nbytes(n, G), dtype=torch.uint8, device=dev)
        codes, scales = ops.split_payload(payload, n, G)
        bound = ops.bind_quant_pack(x, codes, scales)
        host, wall = host_and_wall(lambda i: bound(), 300)
        host_row("one pre-bound launch (quantize+pack of the bucket)", host, wall)
        # the config-5 launch sequence (64 buckets): eager pre-bound launches against one graph replay
        count = 64
        shard = n // world
        stride = -(-ops.payload_nbytes(shard, G) // 256) * 256
        grads = gen(SEED + 7200, count * n, 1e-3, torch.bfloat16)
        residuals = gen(SEED + 7300, count * n, 1e-5)
        rows = torch.empty(world, stride, dtype=torch.uint8, device=dev)
        received = [ops.quant_pack(gen(SEED + 7400 + r, shard, 1e-3), group_size=G) for r in range(world)]
        out = torch.empty(shard, device=dev)
        launches = []
        for i in range(count):
            piece = slice(i * n, (i + 1) * n)
            launches.append(ops.bind_quant_pack_chunks(grads[piece], rows, world, residual=residuals[piece],
                                                       new_residual=residuals[piece]))
            launches.append(ops.bind_dequant_reduce(received, out, numel=shard))

        def eager(_i=0):
            for launch in launches:
                launch()

        host, wall = host_and_wall(eager, 5)
        host_row("64 buckets x (EF quant-pack 8 chunks + W=8 shard reduce), eager pre-bound launches, per bucket",
                 host / count, wall / count)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=torch.cuda.Stream()):
            eager()
        host, wall = host_and_wall(lambda i: graph.replay(), 5)
        host_row("the same sequence as one HIP-graph replay, per bucket", host / count, wall / count)
        # one launch per bucket, the buckets dealt to two streams in turn (a send matrix and an output per lane)
        from lowbit_comm_amd.hip.lanes import StreamLanes

        lanes = StreamLanes(2, dev)
        lane_rows = [rows, torch.empty_like(rows)]
        lane_outs = [out, torch.empty_like(out)]
        steps, previous = [], None
        for i in range(count):
            piece = slice(i * n, (i + 1) * n)
            quant = ops.bind_quant_pack_chunks(grads[piece], lane_rows[i & 1], world, residual=residuals[piece],
                                               new_residual=residuals[piece])
            reduce = ops.bind_dequant_reduce(received, lane_outs[i & 1], numel=shard)
            steps.append(quant if previous is None else ops.bind_quant_chunks_and_reduce(quant, previous))
            previous = reduce

        def two_lanes(_i=0):
            lanes.fork()
            for k, launch in enumerate(steps):
                launch(lanes.handle(k))
            previous(lanes.handle(count))
            lanes.join()

        host, wall = host_and_wall(two_lanes, 5)
        host_row("64 buckets x one launch (EF quant-pack of bucket k + shard reduce of bucket k-1) on two streams in turn, "
                 "eager, per bucket", host / count, wall / count)
        lane_graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(lane_graph, stream=torch.cuda.Stream()):
            two_lanes()
        host, wall = host_and_wall(lambda i: lane_graph.replay(), 5)
        host_row("the same two-stream sequence as one HIP-graph replay, per bucket", host / count, wall / count)
        del grads, residuals, launches, graph, steps, lane_graph

    # ------------------------------------------------------------------------------------------ 8
    if 8 in wanted:
        from lowbit_comm_amd.hip.ring import make_pipelined_ring_executor

        for label, n, dtype, sets_n in (("fp32 chunk of 6,553,600 (200 MiB bucket / 8)", 6_553_600, torch.float32, 8),
                                        ("bf16 chunk of 1,638,400 (25 MiB bucket / 8)", 1_638_400, torch.bfloat16, 24),
                                        ("fp32 chunk of 26,214,400 (a size past the launch ramp-up)", 26_214_400,
                                         torch.float32, 4),
                                        ("bf16 chunk of 52,428,800 (a size past the launch ramp-up)", 52_428_800,
                                         torch.bfloat16, 3)):
            eb = 4 if dtype == torch.float32 else 2
            pb = ops.payload_nbytes(n, G)
            # at least 700 MB between two uses of a buffer: a rotation of one and a half times the 256 MiB memory-side
            # cache is still partly served by it (plain stores are absorbed, the figures read up to 15 % better)
            sets_n = max(sets_n, -(-700_000_000 // (n * eb + 2 * pb)))
            sets = []
            for k in range(sets_n):
                received = torch.empty(pb, dtype=torch.uint8, device=dev)
                ops.quant_pack_payload_into(gen(SEED + 8000 + k, n, 1e-3), received)
                chunk = gen(SEED + 8100 + k, n, 1e-3, dtype)
                send = torch.empty(pb, dtype=torch.uint8, device=dev)
                codes, scales = ops.split_payload(send, n, G)
                sets.append({
                    "chunk": chunk, "send": send, "received": received,
                    "sum": ops.bind_ring_step(received, chunk, send, reduce_op="sum"),
                    "mean": ops.bind_ring_step(received, chunk, send, reduce_op="sum", divisor=8.0),
                    "copy": ops.bind_ring_step(received, chunk, send, reduce_op="none"),
                    "last": ops.bind_ring_step(received, chunk, None, reduce_op="none"),
                    "decode_sum": ops.bind_dequant(*ops.split_payload(received, n, G), chunk, reduce_op="sum"),
                    "quant": ops.bind_quant_pack(chunk, codes, scales),
                })
            check = None
            if parity:
                from oracle import ring_np

                small = 64 * 1000 + 7
                incoming = torch.empty(ops.payload_nbytes(small, G), dtype=torch.uint8, device=dev)
                ops.quant_pack_payload_into(gen(SEED + 8200, small, 1e-3), incoming)
                piece = gen(SEED + 8201, small, 1e-3, dtype)
                before = piece.cpu()
                before = before.view(torch.int16).numpy().view("uint16") if dtype == torch.bfloat16 else before.numpy()
                out_payload = torch.empty_like(incoming)
                ops.ring_step_into(incoming, piece, out_payload, reduce_op="sum", divisor=8.0)
                raw_in = incoming.cpu().numpy()
                groups = ops.num_groups(small, G)
                want, (w_codes, w_scales) = ring_np.ring_step(
                    (raw_in[:groups * G].view("int8"), raw_in[groups * G:].view("float32")), before,
                    "bf16" if dtype == torch.bfloat16 else "fp32", G, reduce_op="sum", divisor=8.0)
                got = piece.cpu()
                got = got.view(torch.int16).numpy().view("uint16") if dtype == torch.bfloat16 else got.numpy().view("uint32")
                ok = bool((got == (want if dtype == torch.bfloat16 else want.view("uint32"))).all())
                raw_out = out_payload.cpu().numpy()
                ok = ok and bool((raw_out[:groups * G].view("int8") == w_codes).all())
                ok = ok and bool((raw_out[groups * G:].view("uint32") == w_scales.view("uint32")).all())
                # full size: the fused launch against the separate ones
                a, b = sets[0], sets[1]
                b["chunk"].copy_(a["chunk"]); b["received"].copy_(a["received"])
                a["sum"](); b["decode_sum"](); b["quant"]()
                ok = ok and bits_equal(a["chunk"], b["chunk"]) and torch.equal(a["send"], b["send"])
                check = "bit-exact" if ok else "MISMATCH"
            payload_bytes = pb
            fused_bytes = 2 * payload_bytes + 2 * n * eb
            emit(8, f"ring step, {label}: decode + accumulate + requantize, one launch", fused_bytes,
                 timed(lambda i: sets[i % sets_n]["sum"](), args.iters * 2), n * eb, check)
            emit(8, f"ring step, {label}: the same with the mean (last reduce hop)", fused_bytes,
                 timed(lambda i: sets[i % sets_n]["mean"](), args.iters * 2), n * eb, check)
            emit(8, f"ring step, {label}: decode + requantize (gather hop)", 2 * payload_bytes + n * eb,
                 timed(lambda i: sets[i % sets_n]["copy"](), args.iters * 2), n * eb, check)
            emit(8, f"ring step, {label}: decode only (last gather hop)", payload_bytes + n * eb,
                 timed(lambda i: sets[i % sets_n]["last"](), args.iters * 2), n * eb, check)

            def separate(i):
                sets[i % sets_n]["decode_sum"]()
                sets[i % sets_n]["quant"]()

            emit(8, f"ring step, {label}: separate decode-accumulate and quantize launches (the reference's sequence)",
                 (payload_bytes + 2 * n * eb) + (n * eb + payload_bytes), timed(separate, args.iters * 2), n * eb, check)
            del sets

        # the same hop in the CUDA extension's byte format (scales interleaved with the codes, or appended)
        from lowbit_comm_amd.hip import cuda_wire as cw

        for label, n, dtype, sets_n, compact in (
                ("fp32 chunk of 6,553,600", 6_553_600, torch.float32, 8, True),
                ("fp32 chunk of 26,214,400", 26_214_400, torch.float32, 4, True),
                ("bf16 chunk of 13,107,200", 13_107_200, torch.bfloat16, 8, True),
                ("bf16 chunk of 52,428,800", 52_428_800, torch.bfloat16, 3, True),
                ("bf16 chunk of 52,428,800, appended scales", 52_428_800, torch.bfloat16, 3, False)):
            eb = 4 if dtype == torch.float32 else 2
            pb = cw.payload_nbytes(n, dtype)
            sets_n = max(sets_n, -(-700_000_000 // (n * eb + 2 * pb)))      # as above
            sets = []
            for k in range(sets_n):
                received = cw.quant_pack(gen(SEED + 8500 + k, n, 1e-3, dtype), compact=compact)
                chunk = gen(SEED + 8600 + k, n, 1e-3, dtype)
                send = torch.empty(pb, dtype=torch.uint8, device=dev)
                sets.append({"chunk": chunk, "send": send, "received": received,
                             "sum": cw.bind_ring_step(received, chunk, send, reduce_op="sum", compact=compact),
                             "copy": cw.bind_ring_step(received, chunk, send, reduce_op="none", compact=compact),
                             "decode_sum": cw.bind_dequant(received, chunk, reduce_op="sum", compact=compact),
                             "quant": cw.bind_quant_pack(chunk, send, compact=compact)})
            check = None
            if parity:
                a, b = sets[0], sets[1]
                b["chunk"].copy_(a["chunk"]); b["received"].copy_(a["received"])
                a["sum"](); b["decode_sum"](); b["quant"]()
                check = "bit-exact vs separate launches" if bits_equal(a["chunk"], b["chunk"]) and torch.equal(a["send"], b["send"]) else "MISMATCH"
            emit(8, f"ring step in the CUDA byte format, {label}: decode + accumulate + requantize, one launch",
                 2 * pb + 2 * n * eb, timed(lambda i: sets[i % sets_n]["sum"](), args.iters * 2), n * eb, check)
            emit(8, f"ring step in the CUDA byte format, {label}: decode + requantize (gather hop)",
                 2 * pb + n * eb, timed(lambda i: sets[i % sets_n]["copy"](), args.iters * 2), pb, check)

            def separate_wire(i):
                sets[i % sets_n]["decode_sum"]()
                sets[i % sets_n]["quant"]()

            emit(8, f"ring step in the CUDA byte format, {label}: separate decode-accumulate and quantize launches",
                 (pb + 2 * n * eb) + (n * eb + pb), timed(separate_wire, args.iters * 2), n * eb, check)
            del sets

        # one rank's whole schedule (W=8, 200 MiB fp32 bucket) through the executor, replaying the bucket's plan
        world, n = 8, 52_428_800
        peer_payload = torch.empty(ops.payload_nbytes(n // world, G), dtype=torch.uint8, device=dev)
        ops.quant_pack_payload_into(gen(SEED + 8300, n // world, 1e-3), peer_payload)

        class Arrived:
            def query(self):
                return True

            def wait_stream(self, s):
                return None

        placed = set()

        def exchange(payload, received, *, send_peer, recv_peer, stream):
            # The link is not part of this measurement: a peer's payload is placed in every receive buffer once.
            if received.data_ptr() not in placed:
                with torch.cuda.stream(stream):
                    received.copy_(peer_payload, non_blocking=True)
                placed.add(received.data_ptr())
            return Arrived()

        buckets = [gen(SEED + 8400 + k, n, 1e-3) for k in range(3)]
        for fused, graphed, inline in ((True, False, False), (True, False, True), (True, True, False), (True, True, True),
                                       (False, False, False)):
            executor = make_pipelined_ring_executor(config=cfg, dtype="fp32", numel=n, world_size=world, rank=3,
                                                    exchange=exchange, fuse_steps=fused, graph_replay=graphed,
                                                    stream=stream if inline else None)

            def whole(i, executor=executor):
                executor.run(buckets[i % 3]).wait()

            for i in range(6):          # per bucket: the run that records its launches, then the run that captures them
                whole(i)
            torch.cuda.synchronize()
            count = 12
            t0 = time.perf_counter()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            for i in range(count):
                whole(i)
            b.record(stream)
            host = (time.perf_counter() - t0) / count
            torch.cuda.synchronize()
            seconds = a.elapsed_time(b) * 1e-3 / count
            chunk_bytes, pay = n // world * 4, ops.payload_nbytes(n // world, G)
            if fused:   # first quantize, 6 sum hops, 1 mean hop, 6 gather hops with payload, 1 without; 14 arrivals
                nbytes = (chunk_bytes + pay) + 7 * (2 * pay + 2 * chunk_bytes) + 6 * (2 * pay + chunk_bytes) + (pay + chunk_bytes)
            else:       # 14 quantize, 7 decode-accumulate, 1 division, 7 decode
                nbytes = 14 * (chunk_bytes + pay) + 7 * (pay + 2 * chunk_bytes) + 2 * chunk_bytes + 7 * (pay + chunk_bytes)
            emit(8, f"one rank's ring schedule, W=8, 200 MiB fp32 bucket, {'fused ring steps' if fused else 'separate launches'}"
                    f"{', replayed as one HIP graph' if graphed else ''}"
                    + (", on the caller's own stream" if inline else "") +
                    f" (14 hops through the executor, payloads of a peer already in the receive buffers; host "
                    f"{host * 1e6:.0f} us per bucket)", nbytes, seconds, n * 4, None)
        del buckets

    print(f"\n{'cfg':>3} {'us':>10} {'GB/s alg.':>10} {'% of 8TB/s':>10} {'input GB/s':>10}  parity / op", file=sys.stderr)
    for r in rows_out:
        if "host_us" in r:
            print(f"{r['config']:>3} {r['us']:10.2f} {'host us':>10} {r['host_us']:10.2f} {'':>10}  {r['op']}", file=sys.stderr)
            continue
        print(f"{r['config']:>3} {r['us']:10.2f} {r['achieved_GBps']:10.1f} {r['frac_of_hbm_peak'] * 100:10.1f} "
              f"{r['input_GBps']:10.1f}  [{r['parity']}] {r['op']}", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
