"""Two guards on the GPU: every entry point of the C ABI is exactly one kernel launch, and the hot-path launches
have not become slower than the frozen baseline.

The reference holds its fused executor to the same two things: one fused kernel per call
(tests/cuda/test_fused_dequant_reduce_mean_ef.py:547-563) and a regression budget against a frozen manifest with
baseline and candidate timed in alternation (tests/benchmarks/fused_dequant_executor_gate.py:16-33,86-90,
tests/benchmarks/baseline_manifest.json).  Here the manifest is profiles/baseline_manifest.json, written by
``python3 bench_configs.py --write-manifest``; what is compared is each launch's time relative to a plain 100 MiB
device copy timed around it in A-B-B-A order in the same run, which takes the box and its clocks out of the
number.  ``LBC_PERF_BUDGET`` (default: the manifest's 0.05) widens or narrows the budget.
"""
import json
import os
from pathlib import Path

import pytest
import torch

# the launch-count test is exact and belongs to the parity suite; the timing gate has a marker of its own

ROOT = Path(__file__).resolve().parent.parent


def kernel_names(run):
    """Names of the device kernels launched while ``run()`` executes, from the profiler's device activity."""
    from torch.profiler import ProfilerActivity, profile

    torch.cuda.synchronize()
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        run()
        torch.cuda.synchronize()
    return [e.name for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA and "Memcpy" not in e.name
            and "Memset" not in e.name]


@pytest.mark.gpu
def test_every_entry_point_is_exactly_one_kernel_launch(hip_device):
    from lowbit_comm_amd.hip import cuda_wire, ops

    dev = hip_device
    n, world, g = 64 * 8 * 100 + 24, 8, 64                     # ragged: interior and edge blocks in one launch
    shard = -(-n // world)
    x = torch.randn(n, device=dev) * 1e-3
    half = x.bfloat16()
    residual = torch.randn(n, device=dev) * 1e-5
    codes, scales = ops.quant_pack(x)
    rows = torch.empty(world, -(-ops.payload_nbytes(shard) // 256) * 256, dtype=torch.uint8, device=dev)
    out = torch.empty(n, device=dev)
    peers = [ops.quant_pack(torch.randn(n, device=dev) * 1e-3) for _ in range(world)]
    requant = (torch.empty_like(codes), torch.empty_like(scales))
    packed = torch.cat([codes.view(torch.uint8), scales.view(torch.uint8)])
    send = torch.empty_like(packed)
    gathered = torch.empty(world * shard, device=dev)
    aligned = 64 * 8 * 100
    quant_chunks = ops.bind_quant_pack_chunks(half[:aligned], rows, world, residual=residual[:aligned],
                                              new_residual=residual[:aligned])
    reduce_shard = ops.bind_dequant_reduce(peers, out)
    wire = cuda_wire.quant_pack(x)
    wire_rows = torch.empty(world, cuda_wire.payload_nbytes(shard, x.dtype), dtype=torch.uint8, device=dev)
    wire_peers = [cuda_wire.quant_pack(torch.randn(n, device=dev) * 1e-3) for _ in range(world)]
    whole = x[:aligned].clone()
    general = torch.empty(cuda_wire.general_payload_nbytes(aligned, x.dtype, 64, 4, 2), dtype=torch.uint8, device=dev)
    # three stages of a bucket stream: the quantize above, a reduce + requantize and a decode in the bucket's type
    part = aligned // world
    arrived = [ops.quant_pack(torch.randn(part, device=dev) * 1e-3) for _ in range(world)]
    mine = ops.quant_pack(torch.zeros(part, device=dev))
    shards = torch.zeros_like(rows)
    assert ops.quant_pack_chunks_into(half[:aligned], shards, world)
    decoded = torch.empty(aligned, dtype=half.dtype, device=dev)
    pipeline_step = ops.bind_bucket_pipeline_step(
        quant_chunks, ops.bind_dequant_reduce_quant(arrived, *mine, part, divisor=8.0, mid_dtype=half.dtype),
        ops.bind_dequant_chunks(shards, decoded, part))
    calls = {
        "lbc_quant_pack": lambda: ops.quant_pack_into(x, codes, scales),
        "lbc_quant_pack (error feedback)": lambda: ops.quant_pack_into(half, codes, scales, residual=residual, new_residual=residual),
        "lbc_quant_pack_chunks": lambda: ops.quant_pack_chunks_into(x, rows, world),
        "lbc_dequant": lambda: ops.dequant_into(codes, scales, out),
        "lbc_dequant_chunks": lambda: ops.dequant_chunks_into(rows, gathered, shard),
        "lbc_dequant_reduce": lambda: ops.dequant_reduce_into(peers, out, divisor=8.0),
        "lbc_dequant_reduce (error feedback)": lambda: ops.dequant_reduce_into(peers, out, divisor=8.0, prepared=x, new_residual=residual),
        "lbc_dequant_reduce_quant": lambda: ops.dequant_reduce_quant_into(peers, *requant, n, divisor=8.0),
        "lbc_quant_pack_chunks_and_dequant_reduce": lambda: ops.bind_quant_chunks_and_reduce(quant_chunks, reduce_shard)(),
        "lbc_bucket_pipeline_step": pipeline_step,
        "lbc_ring_step": lambda: ops.ring_step_into(packed, out, send, reduce_op="sum", divisor=8.0),
        "lbc_ef_update": lambda: ops.ef_update_into(x, out, residual),
        "lbc_wire_quant_pack": lambda: cuda_wire.quant_pack_into(x, wire, residual=residual),
        "lbc_wire_quant_pack_chunks": lambda: cuda_wire.bind_quant_pack_chunks(x, wire_rows, world)(),
        "lbc_wire_dequant": lambda: cuda_wire.dequant_into(wire, out),
        "lbc_wire_dequant_chunks": lambda: cuda_wire.bind_dequant_chunks(wire_rows, gathered, shard)(),
        "lbc_wire_dequant_reduce": lambda: cuda_wire.dequant_reduce_into(wire_peers, out, inv_divisor=0.125),
        "lbc_wire_ring_step": lambda: cuda_wire.ring_step_into(cuda_wire.quant_pack(whole), whole, torch.empty_like(cuda_wire.quant_pack(whole))),
        "lbc_wire_quant_general": lambda: cuda_wire.quant_general_into(whole, general, bit=4, quant_type="normal", topk=2),
        "lbc_wire_dequant_general": lambda: cuda_wire.dequant_general_into(general, whole, bit=4, quant_type="normal", topk=2),
    }
    for name, call in calls.items():
        assert call() is True, name                           # warm up: module load, first-use allocations
    for name, call in calls.items():
        if name == "lbc_wire_ring_step":                      # its operands are made by library calls: bind them first
            received, target = cuda_wire.quant_pack(whole), torch.empty_like(cuda_wire.quant_pack(whole))
            call = lambda: cuda_wire.ring_step_into(received, whole, target)
        launched = kernel_names(call)
        ours = [k for k in launched if "lbc" in k]          # some names arrive mangled (_ZN3lbc...)
        assert len(ours) == 1 and len(launched) == 1, f"{name}: {launched}"


@pytest.mark.gpu_perf
def test_hot_path_launches_hold_the_frozen_baseline(hip_device):
    import bench_configs

    manifest = json.loads((ROOT / "profiles" / "baseline_manifest.json").read_text())
    budget = float(os.environ.get("LBC_PERF_BUDGET", manifest["regression_budget"]))
    rows = bench_configs.gate_rows(quads=3)
    over = [name for name, frozen in manifest["rows"].items() if rows[name]["ratio"] / frozen["ratio"] - 1.0 > budget]
    if over:                                                  # one more look, longer, before calling it a regression
        again = bench_configs.gate_rows(quads=6, only=over)
        for name in over:
            if again[name]["ratio"] < rows[name]["ratio"]:
                rows[name] = again[name]
    report = []
    failed = []
    for name, frozen in manifest["rows"].items():
        now = rows[name]
        change = now["ratio"] / frozen["ratio"] - 1.0
        report.append(f"{name}: {now['us']:.2f} us ({now['frac_of_hbm_peak'] * 100:.1f} %), ratio to copy {now['ratio']:.4f} "
                      f"against {frozen['ratio']:.4f} frozen ({change * 100:+.1f} %)")
        if change > budget:
            failed.append(name)
    print("\n".join(report))
    assert not failed, f"slower than the frozen baseline by more than {budget * 100:.0f} %: {failed}\n" + "\n".join(report)
    assert set(rows) == set(manifest["rows"])
