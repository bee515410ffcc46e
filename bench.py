#!/usr/bin/env python3
"""Benchmark of the compression hot path on one MI355X.

One "step" pushes one 100 MiB fp32 gradient bucket through the compressed reduce-scatter hot path
of one rank at simulated world size 8 (the "config 2" workload): quantize+pack the bucket's 8 destination
chunks, and the fused dequant-reduce of the 8 peer payloads of this rank's shard in fixed rank order.
In a stream of buckets the reduce that is ready when bucket k is quantized belongs to bucket k-1, and the
library carries the two in one launch (lbc_quant_pack_chunks_and_dequant_reduce): that launch is the step,
with the quantize on one buffer set and the reduce on the previous one.  `ms_per_step_two_launches` is the same
work as two launches, `ms_per_step_two_streams` the step's launches dealt to two streams in turn (consecutive
steps are independent, so their ramp-up and drain overlap).  Peer payloads are synthesised in HBM before the timed region; there are no collectives.
`value` is GB/s of gradient input consumed per step.

The line also carries, for the kernel of the step, the HBM roofline: algorithmic bytes per launch / average
launch duration measured with HIP events around back-to-back launches on the launch stream; and a CPU
baseline: the torch-op restatement of the reference codec timed on this host for the same step.  `kernels`
adds the same roofline figures for the kernels of the path launched on their own (quantize+pack of the bucket,
shard reduce, full-bucket all-gather-reduce shape, EF quantize); every leg rotates through more than 600 MB of
buffers, so none of them is served by the 256 MiB memory-side cache.

`roofline.traffic` (HBM bytes per launch of that kernel) is not measured by this run: it comes
from profiles/hbm_traffic.json, which `--record-traffic` writes from two rocprofv3 counter runs
(FETCH_SIZE, WRITE_SIZE) of `bench.py --only step,copy_calibration`, each counter scaled by
what it reads for the plain 100 MiB device copy of the same run.  The file remembers a hash of the kernel
sources it was measured on; when they have changed since, `traffic` is null rather than stale.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
    python bench.py --record-traffic FETCH_SIZE.db WRITE_SIZE.db     (rocprofv3 rocpd databases; no GPU needed)
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

HBM_PEAK = 8.0e12          # MI355X published HBM3E bandwidth, bytes/s
BUCKET_NUMEL = 26_214_400  # 100 MiB of fp32
WORLD = 8
GROUP = 64
SEED = 1234
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
# what the kernel of the step is built from
KERNEL_SOURCES = ("bucket_step.hip", "pipeline_step.hip", "step_grid.h", "quant_pack_block.h", "dequant_reduce_block.h",
                  "device_utils.h", "launch.h", "lbc_api.hip")
BATCHES = 5                # every figure is the median of this many timed batches of --steps launches
WARM_SECONDS = 0.05        # launches go on for at least this long before a leg is timed (clocks settle after idling)
SHARD_SETS = 16            # payload sets of the shard-reduce leg: 16 x 41 MB
CPU_SAMPLE_SECONDS = 10.0  # CPU work of the cpu_baseline leg on all threads (half of it again on one thread)


def kernel_sources_hash() -> str:
    import hashlib

    digest = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "lowbit_comm_amd", "csrc", name), "rb") as handle:
            digest.update(handle.read())
    return digest.hexdigest()[:16]


def recorded_traffic():
    """(bytes per launch of the dominant kernel, where it comes from) or (None, why not)."""
    try:
        with open(TRAFFIC_FILE) as handle:
            record = json.load(handle)
    except (OSError, ValueError):
        return None, "profiles/hbm_traffic.json is missing"
    if record.get("kernel_sources_sha256_16") != kernel_sources_hash():
        return None, "profiles/hbm_traffic.json was measured on other kernel sources; record it again"
    return record["bucket_step"]["traffic_bytes"], "profiles/hbm_traffic.json (rocprofv3 FETCH_SIZE + WRITE_SIZE, copy-calibrated)"


def recorded_pipeline_traffic():
    """The same for the three-stage pipeline step, when the record holds it."""
    try:
        with open(TRAFFIC_FILE) as handle:
            record = json.load(handle)
    except (OSError, ValueError):
        return None
    if record.get("kernel_sources_sha256_16") != kernel_sources_hash():
        return None
    return record.get("bucket_pipeline_step", {}).get("traffic_bytes")


def record_traffic(fetch_db: str, write_db: str) -> int:
    """Write profiles/hbm_traffic.json from the rocpd databases of the two counter runs."""
    import sqlite3

    def per_kernel(path, counter):
        """Median counter value per dispatch (KiB) of every kernel, over its dispatches with the largest grid (the
        set-up phase launches the same quantize kernel on single chunks)."""
        cur = sqlite3.connect(path).cursor()
        tables = [r[0] for r in cur.execute("select name from sqlite_master where type='table'")]
        pick = lambda part: next(t for t in tables if part in t)
        rows = cur.execute(
            f"select s.kernel_name, d.grid_size_x * d.grid_size_y, p.value from {pick('pmc_event')} p "
            f"join {pick('info_pmc')} i on p.pmc_id = i.id join {pick('kernel_dispatch')} d on p.event_id = d.event_id "
            f"join {pick('kernel_symbol')} s on d.kernel_id = s.id where i.name = ?", (counter,)).fetchall()
        largest = {}
        for name, grid, _ in rows:
            largest[name] = max(largest.get(name, 0), grid)
        out = {}
        for name, grid, value in rows:
            if grid == largest[name]:
                out.setdefault(name, []).append(value)
        return {name: sorted(values)[len(values) // 2] for name, values in out.items()}

    fetch, write = per_kernel(fetch_db, "FETCH_SIZE"), per_kernel(write_db, "WRITE_SIZE")
    find = lambda table, part: next(v for k, v in table.items() if part in k)
    copy_kib = BUCKET_NUMEL * 4 / 1024
    fetch_factor, write_factor = copy_kib / find(fetch, "copyBuffer.kd"), copy_kib / find(write, "copyBuffer.kd")
    step_kernel = "bucket_step_kernelIfvLi4EfLi8ELi2E"     # mangled <float, void, 4 per lane, float, 8 payloads, streaming>
    step_fetch, step_write = find(fetch, step_kernel), find(write, step_kernel)
    traffic = (step_fetch * fetch_factor + step_write * write_factor) * 1024
    shard = BUCKET_NUMEL // WORLD
    payload = shard // GROUP * (GROUP + 4)
    pipeline_kernel = "bucket_pipeline_step_kernelIfvLi4ELi8ELi2E"   # mangled <float, void, 4 per lane, 8 payloads, streaming>
    pipe_fetch, pipe_write = find(fetch, pipeline_kernel), find(write, pipeline_kernel)
    record = {
        "kernel_sources_sha256_16": kernel_sources_hash(), "kernel_sources": list(KERNEL_SOURCES),
        "commands": ["rocprofv3 --pmc FETCH_SIZE -d <dir> -o f -- python3 bench.py --steps 20 --warmup 2 --only step,bucket_pipeline_step,copy_calibration",
                     "rocprofv3 --pmc WRITE_SIZE -d <dir> -o w -- python3 bench.py --steps 20 --warmup 2 --only step,bucket_pipeline_step,copy_calibration",
                     "python3 bench.py --record-traffic <dir>/f_results.db <dir>/w_results.db"],
        "calibration": {"kernel": "__amd_rocclr_copyBuffer of 100 MiB (102400 KiB read, 102400 KiB written)",
                        "FETCH_SIZE_factor": fetch_factor, "WRITE_SIZE_factor": write_factor},
        "bucket_step": {"kernel": "bucket_step_kernel<float, void, 4, float, 8, 2>: quantize+pack of a 100 MiB fp32 bucket as 8 "
                                  "chunks and the W=8 reduce of a 3,276,800-element shard in one launch",
                        "FETCH_SIZE_KiB_median": step_fetch, "WRITE_SIZE_KiB_median": step_write,
                        "traffic_bytes": round(traffic),
                        "algorithmic_bytes": BUCKET_NUMEL * 4 + WORLD * payload + WORLD * payload + shard * 4},
        "bucket_pipeline_step": {"kernel": "bucket_pipeline_step_kernel<float, void, 4, 8, 2>: quantize+pack of a 100 MiB fp32 bucket as "
                                           "8 chunks, W=8 reduce + requantize of a 3,276,800-element shard and decode of 8 shard "
                                           "payloads into a 100 MiB bucket in one launch",
                                 "FETCH_SIZE_KiB_median": pipe_fetch, "WRITE_SIZE_KiB_median": pipe_write,
                                 "traffic_bytes": round((pipe_fetch * fetch_factor + pipe_write * write_factor) * 1024),
                                 "algorithmic_bytes": BUCKET_NUMEL * 4 + WORLD * payload + (WORLD + 1) * payload
                                                      + WORLD * payload + BUCKET_NUMEL * 4},
    }
    with open(TRAFFIC_FILE, "w") as handle:
        json.dump(record, handle, indent=1)
        handle.write("\n")
    print(json.dumps(record["bucket_step"]))
    return 0


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sets", type=int, default=6, help="distinct buffer sets rotated through (defeats the LLC)")
    ap.add_argument("--deep-sets", type=int, default=24,
                    help="buffer sets of the deep-rotation legs (0 leaves them out); every set holds 0.5 GB")
    ap.add_argument("--wide-sets", type=int, default=2,
                    help="buffer sets of the whole-bucket reduce (0.33 GB a set) and error-feedback (0.58 GB a set) legs")
    ap.add_argument("--wide-deep-sets", type=int, default=6,
                    help="buffer sets of those two legs' deep-rotation variants (0 leaves them out)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only", default="", help="comma list of kernel legs to time (for profiling one kernel)")
    ap.add_argument("--record-traffic", nargs=2, metavar=("FETCH_DB", "WRITE_DB"),
                    help="write profiles/hbm_traffic.json from two rocprofv3 counter databases and exit")
    return ap.parse_args()


def main() -> int:
    args = parse_args()
    if args.record_traffic:
        return record_traffic(*args.record_traffic)
    if args.gpus != 1:
        print(f"bench.py measures one GPU's share of the path; --gpus {args.gpus} is not supported "
              "(this build has no collectives or multi-GPU sharding)", file=sys.stderr)
        return 2

    import torch

    from lowbit_comm_amd.hip import ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream(dev)

    n, world, g = BUCKET_NUMEL, WORLD, GROUP
    shard = n // world
    payload_bytes = ops.payload_nbytes(shard, g)
    stride = (payload_bytes + 255) // 256 * 256
    only = {k for k in args.only.split(",") if k}

    def gen(seed, numel, sigma, dtype=torch.float32):
        gen_ = torch.Generator(device=dev).manual_seed(seed)
        return (torch.randn(numel, generator=gen_, device=dev) * sigma).to(dtype)

    # ---- synthetic inputs, resident in HBM before any timing -----------------------------------
    def make_set(s):
        bucket = gen(SEED + 100 * s, n, 1e-3)                       # this rank's bucket
        sent = torch.empty(world, stride, dtype=torch.uint8, device=dev)
        received = torch.empty(world, stride, dtype=torch.uint8, device=dev)
        for r in range(world):                                      # peer r's chunk for this rank's shard
            peer_chunk = gen(SEED + 100 * s + 1 + r, shard, 1e-3)
            assert ops.quant_pack_payload_into(peer_chunk, received[r, :payload_bytes], group_size=g)
        out = torch.empty(shard, dtype=torch.float32, device=dev)
        pairs = [ops.split_payload(received[r, :payload_bytes], shard, g) for r in range(world)]
        return {
            "bucket": bucket, "sent": sent, "received": received, "out": out,
            "quant": ops.bind_quant_pack_chunks(bucket, sent, world, group_size=g),
            "reduce": ops.bind_dequant_reduce(pairs, out, group_size=g),
        }

    def add_plan_stages(s):
        """The stages of the reduce-scatter + all-gather plan that follow the quantize, on buffers of this set."""
        s["gathered"] = s["received"].clone()
        s["mine"] = torch.empty(payload_bytes, dtype=torch.uint8, device=dev)
        s["decoded"] = torch.empty(n, dtype=torch.float32, device=dev)
        s["reduce_requant"] = ops.bind_dequant_reduce_quant(
            [ops.split_payload(s["received"][r, :payload_bytes], shard, g) for r in range(world)],
            *ops.split_payload(s["mine"], shard, g), shard, group_size=g, divisor=float(world))
        s["decode"] = ops.bind_dequant_chunks(s["gathered"], s["decoded"], shard, group_size=g)

    sets = [make_set(s) for s in range(args.sets)]
    # the step: the quantize of one set's bucket and the reduce of the previous set's payloads, one launch
    for k, s in enumerate(sets):
        s["step"] = ops.bind_quant_chunks_and_reduce(s["quant"], sets[k - 1]["reduce"])
    torch.cuda.synchronize()

    def step(i):
        if not sets[i % len(sets)]["step"]():
            raise RuntimeError("the library has no shared launch for this quantize and reduce")

    def step_two_launches(i):
        sets[i % len(sets)]["quant"]()
        sets[i % len(sets) - 1]["reduce"]()

    class Seconds(float):
        """Median of the timed batches, in seconds per call; ``low`` and ``high`` are the fastest and slowest batch."""

        low = high = None

    def spread(per_call):
        ordered = sorted(per_call)
        value = Seconds(ordered[len(ordered) // 2])
        value.low, value.high = ordered[0], ordered[-1]
        return value

    def warm(fn, warmup):
        """`warmup` calls and at least WARM_SECONDS of calls: the memory clock of an idle GPU takes tens of
        milliseconds to come up, and a 20-step warm-up is over in well under one."""
        begun, i = time.perf_counter(), 0
        while i < warmup or time.perf_counter() - begun < WARM_SECONDS:
            fn(i)
            i += 1
            if i % 64 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()

    def timed(fn, count, warmup):
        """Seconds per call: BATCHES batches of exactly `count` calls, each bracketed by events on the launch stream
        and a device synchronisation on both sides."""
        warm(fn, warmup)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        per_call = []
        for _ in range(BATCHES):
            start.record(stream)
            for i in range(count):
                fn(i)
            stop.record(stream)
            torch.cuda.synchronize()
            per_call.append(start.elapsed_time(stop) * 1e-3 / count)
        return spread(per_call)

    def timed_on_lanes(fn, lanes, count, warmup):
        """The same for calls dealt to the streams of `lanes` in turn (``fn(i, handle)``).  The lanes are forked from
        the launch stream once, before the warm-up; a batch is bracketed by one event pair per lane and lasts from the
        earliest start to the latest stop, so no fork, join or stream creation falls inside a timed region."""
        lanes.fork()
        warm(lambda i: fn(i, lanes.handle(i)), warmup)
        starts = [torch.cuda.Event(enable_timing=True) for _ in lanes.streams]
        stops = [torch.cuda.Event(enable_timing=True) for _ in lanes.streams]
        per_call = []
        for _ in range(BATCHES):
            for event, lane in zip(starts, lanes.streams):
                event.record(lane)
            for i in range(count):
                fn(i, lanes.handle(i))
            for event, lane in zip(stops, lanes.streams):
                event.record(lane)
            torch.cuda.synchronize()
            per_call.append(max(a.elapsed_time(b) for a in starts for b in stops) * 1e-3 / count)
        lanes.join()
        torch.cuda.synchronize()
        return spread(per_call)

    def milliseconds(seconds):
        return {"median": seconds * 1e3, "min": seconds.low * 1e3, "max": seconds.high * 1e3}

    # ---- the step ---------------------------------------------------------------------------------
    result = {}
    if not only or "step" in only:
        seconds = timed(step, args.steps, args.warmup)
        result["ms_per_step"] = seconds * 1e3
        result["ms_per_step_spread"] = milliseconds(seconds)
        result["value"] = n * 4 / seconds / 1e9
        two = timed(step_two_launches, args.steps, args.warmup)
        result["ms_per_step_two_launches"] = two * 1e3
        result["ms_per_step_two_launches_spread"] = milliseconds(two)
        if len(sets) % 2 == 0:
            # Consecutive steps touch different buffer sets, so they may also be dealt to two streams in turn: the
            # ramp-up of one launch then overlaps the drain of the one before.  Reported next to the headline, which
            # stays on one stream so that a step is one kernel's duration.
            from lowbit_comm_amd.hip.lanes import StreamLanes

            def step_on(i, handle):
                if not sets[i % len(sets)]["step"](handle):
                    raise RuntimeError("the library has no shared launch for this quantize and reduce")

            lanes = timed_on_lanes(step_on, StreamLanes(2, dev), args.steps, args.warmup)
            result["ms_per_step_two_streams"] = lanes * 1e3
            result["ms_per_step_two_streams_spread"] = milliseconds(lanes)

    # ---- per-kernel launch durations ---------------------------------------------------------------
    kernels = {}

    def wanted(name):
        return not only or name in only or ("deep_rotation" in only and name.endswith("_deep_rotation"))

    def leg(name, fn, algorithmic_bytes, launches=None, warmup=None):
        if not wanted(name):
            return
        launches = launches or args.steps
        seconds = timed(fn, launches, warmup if warmup is not None else args.warmup)
        kernels[name] = {
            "us_per_launch": seconds * 1e6, "us_min": seconds.low * 1e6, "us_max": seconds.high * 1e6,
            "algorithmic_bytes": algorithmic_bytes,
            "achieved_GBps": algorithmic_bytes / seconds / 1e9, "frac_of_hbm_peak": algorithmic_bytes / seconds / HBM_PEAK,
        }

    quant_bytes = n * 4 + world * payload_bytes
    reduce_bytes = world * payload_bytes + shard * 4
    if "ms_per_step" in result:
        seconds = result["ms_per_step"] * 1e-3
        spread_ms = result["ms_per_step_spread"]
        kernels["bucket_step"] = {
            "us_per_launch": seconds * 1e6, "us_min": spread_ms["min"] * 1e3, "us_max": spread_ms["max"] * 1e3,
            "algorithmic_bytes": quant_bytes + reduce_bytes,
            "achieved_GBps": (quant_bytes + reduce_bytes) / seconds / 1e9,
            "frac_of_hbm_peak": (quant_bytes + reduce_bytes) / seconds / HBM_PEAK,
        }
    leg("quant_pack_chunks", lambda i: sets[i % len(sets)]["quant"](), quant_bytes)
    if not only or "bucket_pipeline_step" in only or "pipeline_three_launches" in only:
        # the whole reduce-scatter + all-gather plan as the drop-in transport runs it on a stream of buckets: one launch
        # carries the quantize of bucket k, the reduce + requantize of the payloads that arrived for bucket k-1 and the
        # decode of the gathered shard payloads of bucket k-2 into that bucket (lbc_bucket_pipeline_step)
        for s in sets:
            add_plan_stages(s)
        for k, s in enumerate(sets):
            s["pipeline_step"] = ops.bind_bucket_pipeline_step(s["quant"], sets[k - 1]["reduce_requant"], sets[k - 2]["decode"])
        plan_bytes = quant_bytes + (world + 1) * payload_bytes + world * payload_bytes + n * 4

        def pipeline_step(i):
            if not sets[i % len(sets)]["pipeline_step"]():
                raise RuntimeError("the library has no shared launch for these three stages")

        def pipeline_three_launches(i):
            sets[i % len(sets)]["quant"]()
            sets[i % len(sets) - 1]["reduce_requant"]()
            sets[i % len(sets) - 2]["decode"]()

        leg("bucket_pipeline_step", pipeline_step, plan_bytes)
        if "bucket_pipeline_step" in kernels:
            kernels["bucket_pipeline_step"]["traffic"] = recorded_pipeline_traffic()
        leg("pipeline_three_launches", pipeline_three_launches, plan_bytes)
        for s in sets:
            for name in ("gathered", "mine", "decoded", "reduce_requant", "decode", "pipeline_step"):
                del s[name]
        torch.cuda.empty_cache()
    if (wanted("bucket_step_deep_rotation") or wanted("bucket_pipeline_step_deep_rotation")) and args.deep_sets > len(sets):
        # The same two launches with four times as many buffer sets in rotation (4 GB and 7 GB instead of 1 GB and
        # 1.8 GB between two uses of a buffer): launches that write much read a few percent slower this way although
        # the traffic that leaves the L2 is the same, so both figures are in the line.
        deep = sets + [make_set(s) for s in range(len(sets), args.deep_sets)]
        for s in deep:
            add_plan_stages(s)
        deep_steps = [ops.bind_quant_chunks_and_reduce(s["quant"], deep[k - 1]["reduce"]) for k, s in enumerate(deep)]
        deep_plans = [ops.bind_bucket_pipeline_step(s["quant"], deep[k - 1]["reduce_requant"], deep[k - 2]["decode"])
                      for k, s in enumerate(deep)]

        def run_deep(launches):
            def call(i):
                if not launches[i % len(launches)]():
                    raise RuntimeError("the library has no shared launch for these stages")
            return call

        leg("bucket_step_deep_rotation", run_deep(deep_steps), quant_bytes + reduce_bytes, launches=max(args.steps, 48))
        leg("bucket_pipeline_step_deep_rotation", run_deep(deep_plans),
            quant_bytes + (2 * world + 1) * payload_bytes + n * 4, launches=max(args.steps, 48))
        for name in ("bucket_step_deep_rotation", "bucket_pipeline_step_deep_rotation"):
            if name in kernels:
                kernels[name]["buffer_sets"] = len(deep)
        for s in deep:
            for name in ("gathered", "mine", "decoded", "reduce_requant", "decode"):
                del s[name]
        del deep, deep_steps, deep_plans
        torch.cuda.empty_cache()
    if not only or "dequant_reduce_shard" in only:
        # the shard reduce alone moves 41 MB a launch: it gets payload sets of its own, enough of them (656 MB) that
        # no launch finds its operands in the memory-side cache
        shard_sets = []
        for s in range(SHARD_SETS):
            rows = sets[s % len(sets)]["received"].clone()
            out = torch.empty(shard, dtype=torch.float32, device=dev)
            pairs = [ops.split_payload(rows[r, :payload_bytes], shard, g) for r in range(world)]
            shard_sets.append(ops.bind_dequant_reduce(pairs, out, group_size=g))
        # a launch of 8-9 us: batches of at least 96, so that the first launch after the synchronisation (which meets
        # an idle GPU) does not weigh a twentieth of the figure
        leg("dequant_reduce_shard", lambda i: shard_sets[i % SHARD_SETS](), reduce_bytes, launches=max(args.steps, 96))
        del shard_sets
        torch.cuda.empty_cache()

    if not only or "copy_calibration" in only:
        # a plain device copy of known size (100 MiB read + 100 MiB written): scales the HBM counters, and shows
        # what this box sustains on the simplest possible streaming kernel next to the codec kernels
        srcs = [sets[i]["bucket"] for i in range(len(sets))]
        dsts = [torch.empty_like(srcs[0]) for _ in range(2)]
        leg("copy_calibration", lambda i: dsts[i % 2].copy_(srcs[i % len(srcs)]), 2 * n * 4)
        del dsts

    if any(wanted(k + d) for k in ("dequant_reduce_full", "ef_quant_pack") for d in ("", "_deep_rotation")):
        # Both legs are timed twice: over --wide-sets buffer sets (two: 0.66 and 1.16 GB in rotation, past the
        # last-level cache, within what the address-translation caches still cover) and over --wide-deep-sets (six),
        # where every launch also pays for translation misses, as a stream of gradient buckets does.
        def rotations(name):
            for count, suffix in ((args.wide_sets, ""), (args.wide_deep_sets, "_deep_rotation")):
                if count > 0 and (suffix == "" or count > args.wide_sets) and wanted(name + suffix):
                    yield count, name + suffix

        def run_over(launches):
            return lambda i: launches[i % len(launches)]()

        # all-gather-reduce shape: 8 payloads of the whole bucket -> fp32 bucket
        full_sets = []
        for count, name in rotations("dequant_reduce_full"):
            for s in range(len(full_sets), count):
                pairs = [ops.quant_pack(gen(SEED + 7000 + 10 * s + r, n, 1e-3), group_size=g) for r in range(world)]
                out = torch.empty(n, dtype=torch.float32, device=dev)
                full_sets.append(ops.bind_dequant_reduce(pairs, out, group_size=g))
            leg(name, run_over(full_sets[:count]), world * ops.payload_nbytes(n, g) + n * 4,
                launches=max(24, args.steps // 4), warmup=6)
            if name in kernels:
                kernels[name]["buffer_sets"] = count
        del full_sets
        torch.cuda.empty_cache()
        # config 3: 100 MiB bf16 gradient + fp32 residual, residual updated in place
        n3 = 52_428_800
        groups3 = ops.num_groups(n3, g)
        ef_sets = []
        for count, name in rotations("ef_quant_pack"):
            for s in range(len(ef_sets), count):
                grad = gen(SEED + 9000 + s, n3, 1e-3, torch.bfloat16)
                residual = gen(SEED + 9100 + s, n3, 1e-5)
                codes = torch.empty(groups3 * g, dtype=torch.int8, device=dev)
                scales = torch.empty(groups3, dtype=torch.float32, device=dev)
                ef_sets.append(ops.bind_quant_pack(grad, codes, scales, group_size=g, residual=residual,
                                                   new_residual=residual))
            leg(name, run_over(ef_sets[:count]), n3 * (2 + 4 + 4) + groups3 * (g + 4),
                launches=max(24, args.steps // 4), warmup=6)
            if name in kernels:
                kernels[name]["buffer_sets"] = count
        del ef_sets
        torch.cuda.empty_cache()

    # ---- parity of the timed workload + CPU baseline (oracle, checker only) -------------------
    cpu_baseline = None
    parity = None
    if not args.no_cpu_baseline and not only:
        from oracle import codec_torch

        s0 = sets[0]
        if not ops.bind_quant_chunks_and_reduce(s0["quant"], s0["reduce"])():     # the step's launch, on one set
            raise RuntimeError("the library has no shared launch for this quantize and reduce")
        torch.cuda.synchronize()
        bucket_cpu = s0["bucket"].cpu()
        received_cpu = s0["received"].cpu()

        def cpu_step():
            payloads = [codec_torch.quantize(bucket_cpu[d * shard:(d + 1) * shard], g) for d in range(world)]
            peers = []
            for r in range(world):
                row = received_cpu[r, :payload_bytes]
                peers.append((row[:shard].view(torch.int8), row[shard:].view(torch.float32)))
            return payloads, codec_torch.reduce_payloads(peers, shard, g, "fp32", "sum")

        payloads, reduced = cpu_step()
        sent_cpu = s0["sent"].cpu()
        ok = all(torch.equal(sent_cpu[d, :payload_bytes], codec_torch.pack(*payloads[d])) for d in range(world))
        ok = ok and torch.equal(s0["out"].cpu().view(torch.int32), reduced.view(torch.int32))
        parity = "bit-exact" if ok else "MISMATCH"
        # A bounded sample of the same step: repeats for about ten seconds of CPU work, so that the figure is the
        # host's steady state and not that of a cold thread pool (hosts still differ: 2.0 to 14 GB/s were seen).
        times = []
        deadline = time.perf_counter() + CPU_SAMPLE_SECONDS
        while len(times) < 3 or (time.perf_counter() < deadline and len(times) < 5000):
            t0 = time.perf_counter()
            cpu_step()
            times.append(time.perf_counter() - t0)
        times = sorted(times[3:] or times)
        median = times[len(times) // 2]
        threads = torch.get_num_threads()
        single = None
        if threads > 1:                                   # the same step on one thread, a few repeats
            torch.set_num_threads(1)
            one = []
            stop_at = time.perf_counter() + CPU_SAMPLE_SECONDS / 2
            while len(one) < 2 or (time.perf_counter() < stop_at and len(one) < 1000):
                t0 = time.perf_counter()
                cpu_step()
                one.append(time.perf_counter() - t0)
            torch.set_num_threads(threads)
            one = sorted(one[1:] or one)
            single = one[len(one) // 2]
        model = "unknown"
        try:
            with open("/proc/cpuinfo") as info:
                model = next((line.split(":", 1)[1].strip() for line in info if line.startswith("model name")), model)
        except OSError:
            pass
        cpu_baseline = {
            "value": n * 4 / median / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{len(times)} timed repeats ({sum(times):.1f} s) of the full step (8x quantize of 3,276,800-element "
                      f"chunks + 8-payload left-fold reduce of one shard) with torch CPU ops, median {median * 1e3:.1f} ms; "
                      f"host has {os.cpu_count()} logical CPUs",
            "single_thread_value": None if single is None else n * 4 / single / 1e9,
            "cpu_model": model,
        }

    dominant = kernels.get("bucket_step")
    traffic, traffic_source = recorded_traffic()
    line = {
        "metric": "quant-pack & fused dequant-reduce GB/s on 1 MI355X; % of HBM roofline",
        "value": result.get("value"),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "batches": BATCHES,
        "timing": f"every figure is the median of {BATCHES} batches of exactly `steps` launches, each batch bracketed by HIP "
                  f"events and a device synchronisation, after `warmup` launches and at least {WARM_SECONDS * 1e3:.0f} ms of "
                  "launches; *_spread and us_min / us_max give the fastest and slowest batch",
        "ms_per_step": result.get("ms_per_step"),
        "ms_per_step_spread": result.get("ms_per_step_spread"),
        "ms_per_step_two_launches": result.get("ms_per_step_two_launches"),
        "ms_per_step_two_launches_spread": result.get("ms_per_step_two_launches_spread"),
        "ms_per_step_two_streams": result.get("ms_per_step_two_streams"),
        "ms_per_step_two_streams_spread": result.get("ms_per_step_two_streams_spread"),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "config 2: 100 MiB fp32 bucket ~N(0,1e-3 std), W=8, group 64: quant-pack of the 8 chunks + "
                        "fused dequant-reduce of one rank's shard (8 payloads x 3,276,800 codes), fixed rank order; "
                        "one launch carries the quantize of a bucket and the shard reduce of the bucket before it",
            "bucket_numel": n, "world_size": world, "group_size": g, "buffer_sets": args.sets,
            "value_is": "bucket bytes (104,857,600) consumed per step / step time",
        },
        "roofline": None if dominant is None else {
            "bound": "hbm", "kernel": "bucket_step_kernel (quant-pack of the 100 MiB fp32 bucket as 8 chunks + W=8 reduce "
                                      "of one shard, one launch)",
            "achieved": dominant["achieved_GBps"], "peak": HBM_PEAK / 1e9, "unit": "GB/s",
            "frac": dominant["frac_of_hbm_peak"], "traffic": traffic, "traffic_source": traffic_source,
            "algorithmic_bytes": dominant["algorithmic_bytes"], "us_per_launch": dominant["us_per_launch"],
            "buffer_sets": args.sets,
            # the same kernel with four times as many buffer sets in rotation (see kernels.bucket_step_deep_rotation)
            "frac_deep_rotation": kernels.get("bucket_step_deep_rotation", {}).get("frac_of_hbm_peak"),
        },
        "cpu_baseline": cpu_baseline,
        "parity": parity,
        "kernels": kernels,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
