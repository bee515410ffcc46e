"""The C-ABI library loads without a GPU and exports every symbol include/lbc.h declares; plus the exhaustive
host-side proof of the division-free scale formula the quantizer uses."""
import ctypes
import re
import subprocess
from pathlib import Path

import pytest

from lowbit_comm_amd.hip import library

ROOT = Path(__file__).resolve().parent.parent


def declared_functions():
    text = (ROOT / "include" / "lbc.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lbc_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree_on_the_symbol_list():
    assert declared_functions() == sorted(library.SIGNATURES)


def test_library_loads_on_the_cpu_and_exports_every_declared_symbol():
    assert library.LIBRARY_PATH.exists(), "run __graft_entry__.build() first"
    lib = library.load_library()
    for name in declared_functions():
        assert hasattr(lib, name), name
    assert lib.lbc_abi_version() == library.ABI_VERSION


def test_argument_validation_happens_before_any_device_work():
    lib = library.load_library()
    none = ctypes.c_void_p(None)
    assert lib.lbc_quant_pack(none, 0, none, -1, -5, 64, none, none, none, -1, none, 0, none, -1, 0, none) == -1
    assert library.last_error(lib) == "numel must be >= 0"
    assert lib.lbc_quant_pack(none, 7, none, -1, 64, 64, none, none, none, -1, none, 0, none, -1, 0, none) == -1
    assert "unsupported input dtype" in library.last_error(lib)
    assert lib.lbc_quant_pack(none, 0, none, -1, 0, 64, none, none, none, -1, none, 0, none, -1, 0, none) == 0      # empty: no-op
    assert lib.lbc_quant_pack(none, 0, none, -1, 64, 48, none, none, none, -1, none, 0, none, -1, 0, none) == 1     # unsupported group
    assert lib.lbc_dequant_reduce(none, none, 0, 64, 64, 1.0, none, 0, none, none, 0, none) == -1
    assert library.last_error(lib) == "inputs must not be empty"
    assert lib.lbc_dequant_reduce(none, none, 9, 64, 64, 1.0, none, 0, none, none, 0, none) == 1          # > 8 payloads
    assert lib.lbc_dequant_reduce(none, none, 2, 64, 64, 0.0, none, 0, none, none, 0, none) == -1
    assert library.last_error(lib) == "divisor must be > 0"
    assert lib.lbc_quant_pack_chunks(none, 0, none, -1, 640, 0, 64, none, 0, none, -1, none, 0, none, -1, 0, none) == -1
    assert library.last_error(lib) == "world must be > 0"
    assert lib.lbc_dequant(none, none, 64, 64, none, 0, 9, 0, none) == -1
    # ring / tree hops: (recv codes, recv scales, chunk, dtype, numel, g, op, divisor, send codes, send scales, access,
    # stream)
    assert lib.lbc_ring_step(none, none, none, 0, -1, 64, 1, 1.0, none, none, 0, none) == -1
    assert library.last_error(lib) == "numel must be >= 0"
    assert lib.lbc_ring_step(none, none, none, 5, 64, 64, 1, 1.0, none, none, 0, none) == -1
    assert "unsupported chunk dtype" in library.last_error(lib)
    assert lib.lbc_ring_step(none, none, none, 0, 64, 64, 1, 0.0, none, none, 0, none) == -1
    assert library.last_error(lib) == "divisor must be > 0"
    assert lib.lbc_ring_step(none, none, none, 0, 64, 64, 7, 1.0, none, none, 0, none) == -1
    assert "unknown reduce op" in library.last_error(lib)
    assert lib.lbc_ring_step(none, none, none, 0, 64, 64, 2, 1.0, none, none, 0, none) == 1        # MAX: unsupported
    assert lib.lbc_ring_step(none, none, none, 0, 64, 48, 1, 1.0, none, none, 0, none) == 1        # group 48
    assert lib.lbc_ring_step(none, none, none, 0, 0, 64, 1, 1.0, none, none, 0, none) == 0         # empty: no-op
    assert lib.lbc_ring_step(none, none, none, 0, 64, 64, 1, 1.0, none, none, 0, none) == -1
    assert "must not be null" in library.last_error(lib)
    # (received, chunk, dtype, numel, g, compact, op, divisor, send, access, stream)
    assert lib.lbc_wire_ring_step(none, none, 0, 100, 64, 1, 1, 1.0, none, 0, none) == -1
    assert library.last_error(lib) == "numel should be multiple of group_size"
    assert lib.lbc_wire_ring_step(none, none, 0, 128, 64, 1, 3, 1.0, none, 0, none) == 1           # MIN: unsupported
    assert lib.lbc_wire_ring_step(none, none, 0, 0, 64, 1, 1, 1.0, none, 0, none) == 0
    assert lib.lbc_wire_ring_step(none, none, 0, 128, 64, 1, 1, -2.0, none, 0, none) == -1
    # the access mode is an argument of the call (0 auto, 1 cached, 2 stream); there is no process-wide setting
    assert lib.lbc_quant_pack(none, 0, none, -1, 0, 64, none, none, none, -1, none, 0, none, -1, 2, none) == 0
    assert lib.lbc_quant_pack(none, 0, none, -1, 0, 64, none, none, none, -1, none, 0, none, -1, 3, none) == -1
    assert library.last_error(lib) == "unknown access mode 3"
    assert lib.lbc_dequant(none, none, 0, 64, none, 0, 0, -1, none) == -1
    assert not hasattr(lib, "lbc_set_stream_min_bytes")


def test_missing_library_raises_instead_of_falling_back(tmp_path):
    from lowbit_comm_amd import CCDLUnavailableError

    with pytest.raises(CCDLUnavailableError, match="not built"):
        library.load_library(tmp_path / "liblbc_hip.so")


def test_scale_formula_is_exact_for_every_finite_float(tmp_path):
    """absmax/127 computed as q0 = a*c, r = fma(-q0,127,a), q1 = fma(r,c,q0) equals the IEEE division for all
    2^31 - 2^23 non-negative finite floats (about half a minute on 8 cores)."""
    binary = tmp_path / "check_scale127"
    subprocess.run(["gcc", "-O2", "-mfma", "-fopenmp", "-ffp-contract=off", "-o", str(binary),
                    str(ROOT / "tests" / "native" / "check_scale127.c"), "-lm"], check=True)
    done = subprocess.run([str(binary)], capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stdout
    assert "mismatches with result >= 2^-24: 0 ; below (clamped region): 0" in done.stdout
    assert "0x3C010204" in done.stdout


def test_division_free_quotient_matches_the_division_next_to_every_tie(tmp_path):
    """The encode's q1 = fma(fma(-q0, s, p), 1/s, q0) against p / s on the CPU, for dividends within 8 ulps of every
    half-integer and integer multiple of the scale: every scale with at most 11 significant mantissa bits and the
    (almost) all-ones mantissas at the ends and the middle of the scale's exponent range, and four million random
    mantissas (3.6e10 pairs, about 15 s on 8 cores).  The GPU suite walks all 2^23 mantissas on the device."""
    binary = tmp_path / "check_quotient"
    subprocess.run(["gcc", "-O2", "-mfma", "-fopenmp", "-ffp-contract=off", "-o", str(binary),
                    str(ROOT / "tests" / "native" / "check_quotient.c"), "-lm"], check=True)
    done = subprocess.run([str(binary)], capture_output=True, text=True, timeout=900)
    assert done.returncode == 0, done.stdout
    assert "code mismatches 0, quotient mismatches 0" in done.stdout
    assert int(done.stdout.split()[1].rstrip(",")) > 3 * 10 ** 10


def test_code_book_cell_lookup_is_the_search_and_rounding_on_every_float(tmp_path):
    """The code-book quantizer of the CUDA byte format encodes the quotients with one table lookup
    (csrc/code_book_cells.h, tables built at compile time).  For each of the four books and every float in [-1, 1]
    (8.5e9 values, about 15 s on 8 cores) the lookup gives the code of the reference's search and rounding step, and
    every step of the table is checked on both sides whatever the stride."""
    binary = tmp_path / "check_book_cells"
    subprocess.run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-fopenmp", "-o", str(binary),
                    str(ROOT / "tests" / "native" / "check_book_cells.cpp")], check=True)
    done = subprocess.run([str(binary)], capture_output=True, text=True, timeout=900)
    assert done.returncode == 0, done.stdout
    lines = done.stdout.splitlines()
    assert lines[-1] == "MISMATCHES 0" and int(lines[-2].split()[1]) > 8 * 10 ** 9
    assert sum(line.endswith(", 0 mismatches") for line in lines) == 4


def test_sum_of_two_16_bit_values_through_fp32_is_the_native_sum(tmp_path):
    """The CUDA-format kernels add two fp16 / bfloat16 values with one fp32 add and one conversion; for every pair
    of finite values of either type that is the correctly rounded 16-bit sum (about half a minute on 8 cores)."""
    binary = tmp_path / "check_half_sum"
    subprocess.run(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", "-o", str(binary),
                    str(ROOT / "tests" / "native" / "check_half_sum.c"), "-lm"], check=True)
    done = subprocess.run([str(binary)], capture_output=True, text=True, timeout=900)
    assert done.returncode == 0, done.stdout
    assert "fp16: 2015394816 pairs, 0 mismatches" in done.stdout
    assert "bfloat16: 2130771840 pairs, 0 mismatches" in done.stdout


def test_device_code_has_no_instruction_that_changes_the_rounding_contract(tmp_path):
    """The parity argument rests on build flags: products and sums round separately.  Compile the two kernel
    files to assembly with the Makefile's flags and check that no packed-fp32 arithmetic and no
    fused multiply-convert (`v_fma_mix*`, which rounds a product straight to fp16) was selected."""
    makefile = (ROOT / "lowbit_comm_amd" / "csrc" / "Makefile").read_text()
    flags = re.search(r"HIPFLAGS\s*:=\s*((?:.*\\\n)*.*)", makefile).group(1).replace("\\\n", " ").split()
    flags = [f.replace("$(ARCH)", "gfx950") for f in flags if f != "-fPIC"]
    assert "-ffp-contract=off" in flags
    procs = []
    for name in ("quant_pack", "dequant_reduce"):
        out = tmp_path / f"{name}.s"
        procs.append((out, subprocess.Popen(
            ["/opt/rocm/bin/hipcc", *flags, "--cuda-device-only", "-S", str(ROOT / "lowbit_comm_amd" / "csrc" / f"{name}.hip"),
             "-o", str(out)], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)))
    for out, proc in procs:
        assert proc.wait(timeout=900) == 0
        text = out.read_text()
        assert "gfx950" in text
        for forbidden in ("v_fma_mix", "v_mad_mix", "v_pk_mul_f32", "v_pk_add_f32", "v_pk_fma_f32"):
            assert forbidden not in text, (out.name, forbidden)


def test_product_code_never_reaches_into_the_oracle_or_the_working_folder():
    """The oracle is a checker: only tests, the smoke check and the benchmark's CPU-baseline leg may load it."""
    offenders = []
    for path in sorted((ROOT / "lowbit_comm_amd").rglob("*")):
        if path.suffix not in (".py", ".hip", ".h") or "_build" in path.parts:
            continue
        text = path.read_text(errors="ignore")
        if re.search(r"^\s*(from|import)\s+(oracle|_work)\b|\boracle/|\b_work/", text, flags=re.M):
            offenders.append(str(path.relative_to(ROOT)))
    assert offenders == []
    bench = (ROOT / "bench.py").read_text()
    assert "_work/" not in bench and "_work/" not in (ROOT / "__graft_entry__.py").read_text()
