"""The C ABI driven by a host program that has neither Python nor torch in it (tests/native/abi_client.cpp, built by
``__graft_entry__.build()``): HIP runtime allocations, a stream of its own, results compared byte for byte with the
scalar C oracle inside the program."""
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
CLIENT = ROOT / "tests" / "native" / "_build" / "abi_client"


def test_client_source_uses_only_the_header_and_the_hip_runtime():
    text = (ROOT / "tests" / "native" / "abi_client.cpp").read_text()
    includes = [line.split()[1] for line in text.splitlines() if line.startswith("#include")]
    assert '"../../include/lbc.h"' in includes and "<hip/hip_runtime.h>" in includes
    assert not any("torch" in name or "Python" in name or "pybind" in name for name in includes)
    assert CLIENT.exists(), "run __graft_entry__.build() first"


@pytest.mark.gpu
def test_client_runs_every_entry_point_bit_exact_against_the_c_oracles(hip_device):
    """Portable format: quantize, decode, fused reduce, ring step, the error-feedback step and the residual update, the
    bucket as chunks and the chunks decoded back, reduce + requantize, the shared launch of a quantize and a reduce,
    the sum of bucket and residual as an output of the quantize, the three-stage pipeline step, and two contract
    checks (33).  The CUDA extension's byte format: quantize and decode for fp32 / bf16, interleaved /
    appended scales, 8 / 4 bits; fused mean of four payloads; ring step; chunks; four general policies (29)."""
    done = subprocess.run([str(CLIENT)], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, (done.stdout, done.stderr[-2000:])
    assert done.stdout.strip().startswith("OK "), done.stdout
    assert int(done.stdout.split()[1]) == 63


@pytest.mark.gpu
def test_exact_quotient_without_a_division_matches_the_division_on_billions_of_pairs(hip_device):
    """tests/native/quotient_check.hip: the encode's FMA-refined quotient against ``p / s`` on the device.  4.3e9
    pairs in each of six sampled modes (random, extreme scale mantissas, quotients next to ties, 16-bit dividends)
    with scale exponents over the whole domain, and the exhaustive walk over every scale mantissa and every dividend
    next to a half-integer multiple of the scale, the only pairs whose code the refinement could change; and the
    code-book quantizer's division with a shared reciprocal against the division, bit for bit."""
    checker = ROOT / "tests" / "native" / "_build" / "quotient_check"
    assert checker.exists(), "run __graft_entry__.build() first"
    done = subprocess.run([str(checker), "1", "1"], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout[-2000:]
    assert "MISMATCHES 0" in done.stdout.splitlines()[-1]
    assert done.stdout.count("code mismatches 0") == 8 and done.stdout.count("quotient mismatches 0 ") == 8


@pytest.mark.gpu
def test_code_book_cell_lookup_is_the_search_and_rounding_on_the_device(hip_device):
    """tests/native/book_cells_check.hip: the one-lookup code-book encoder of the quantize kernel (the cell of
    fma(t, 128, 128), then ``base + (t >= threshold)``) against the search and rounding it stands for, both on the
    device, for the four books and every float in [-1, 1]."""
    checker = ROOT / "tests" / "native" / "_build" / "book_cells_check"
    assert checker.exists(), "run __graft_entry__.build() first"
    done = subprocess.run([str(checker)], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout[-2000:]
    lines = done.stdout.splitlines()
    assert lines[-1] == "MISMATCHES 0" and int(lines[-2].split()[1]) > 8 * 10 ** 9
