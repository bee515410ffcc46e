"""The hot kernels against do-nothing kernels with their traffic mix, on the GPU.

tests/native/stream_probe.hip moves the same bytes per lane as the W=8 fused reduce (eight dwords of codes, eight
shared scales, one 16-byte store) and as the fp32 quantize (16 bytes in, 4 bytes out) with the same cache hints and
block order, and computes nothing.  What it reaches is the ceiling for the shape, launch ramp included; the codec
kernels, which also convert, multiply, sum and take group maxima with exact quotients, must stay within 0.9 of it.
"""
import subprocess
from pathlib import Path

import pytest
import torch

pytestmark = pytest.mark.gpu_perf      # a timing gate: run with -m gpu_perf, apart from the parity suite

PROBE = Path(__file__).resolve().parent / "native" / "_build" / "stream_probe"
ROTATE = 640_000_000


def probe_rows(reduce_elems, quant_elems):
    done = subprocess.run([str(PROBE), "rows", str(reduce_elems), str(quant_elems)], capture_output=True, text=True,
                          timeout=120, check=True)
    rows = {}
    for line in done.stdout.splitlines():
        if line.startswith("ROW "):
            _, name, us, nbytes = line.split()
            rows[name] = (float(us), int(nbytes))
    return rows


def back_to_back(launches, repeats=10):
    stream = torch.cuda.current_stream()
    for launch in launches:
        launch()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(3):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(repeats):
            for launch in launches:
                launch()
        stop.record(stream)
        stop.synchronize()
        best = min(best, start.elapsed_time(stop) * 1e3 / (repeats * len(launches)))
    return best


@pytest.mark.parametrize("reduce_elems,quant_elems", [(3_276_800, 26_214_400), (26_214_400, 6_553_600)])
def test_reduce_and_quantize_stay_within_a_tenth_of_a_kernel_that_only_moves_their_bytes(hip_device, reduce_elems, quant_elems):
    from lowbit_comm_amd.hip import ops

    assert PROBE.exists(), "run __graft_entry__.build() first"
    rows = probe_rows(reduce_elems, quant_elems)
    dev = hip_device
    world = 8

    def payload(n):
        g = n // 64
        return (torch.randint(-127, 128, (n,), dtype=torch.int8, device=dev), torch.rand(g, device=dev) * 1e-5 + 1e-6)

    reduce_bytes = world * (reduce_elems // 64) * 68 + reduce_elems * 4
    reduces = [ops.bind_dequant_reduce([payload(reduce_elems) for _ in range(world)], torch.empty(reduce_elems, device=dev))
               for _ in range(ROTATE // reduce_bytes + 1)]
    reduce_us = back_to_back(reduces)
    del reduces
    torch.cuda.empty_cache()
    quant_bytes = quant_elems * 4 + (quant_elems // 64) * 68
    quants = []
    for _ in range(ROTATE // quant_bytes + 1):
        codes, scales = payload(quant_elems)
        quants.append(ops.bind_quant_pack(torch.randn(quant_elems, device=dev) * 1e-3, codes, scales))
    quant_us = back_to_back(quants)
    del quants
    torch.cuda.empty_cache()
    probe_reduce_us, probe_quant_us = rows["reduce_like_w8"][0], rows["quant_like_fp32"][0]
    print(f"W=8 reduce of {reduce_elems} elements: {reduce_us:.2f} us, the probe {probe_reduce_us:.2f} us "
          f"({probe_reduce_us / reduce_us:.2f}); fp32 quantize of {quant_elems} elements: {quant_us:.2f} us, the probe "
          f"{probe_quant_us:.2f} us ({probe_quant_us / quant_us:.2f})")
    assert probe_reduce_us / reduce_us >= 0.9
    assert probe_quant_us / quant_us >= 0.9
