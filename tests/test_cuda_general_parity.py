"""GPU parity of the general CUDA-format kernels (code books, stochastic rounding, top-k side channel,
NaN-resetting maximum) against the CPU oracle (oracle/cuda_wire_general_np.py): payload bytes and decoded
values, bit-exact; size-independent properties at the full bucket size."""
from __future__ import annotations

import itertools

import numpy as np
import pytest
import torch

from oracle import cuda_wire_general_np as general
from oracle import cuda_wire_np as wire

from tests.test_cuda_wire_parity import NAMES, from_numpy, same, to_numpy

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip(hip_device):
    from lowbit_comm_amd.hip import cuda_wire

    return cuda_wire


def policies():
    for bit, topk, stochastic in itertools.product((4, 8), (0, 1, 2), (None, (42, 8), (7, 3))):
        for quant_type in (general.QUANT_TYPES if bit == 4 else ("linear",)):
            yield bit, quant_type, topk, stochastic


def awkward_values(rng, n, g, case):
    values = (rng.standard_normal(n) * rng.choice([1e-7, 1e-3, 1.0, 100.0])).astype(np.float32)
    values[rng.integers(0, n, max(1, n // 40))] = 0.0
    values[rng.integers(0, n, max(1, n // 500))] *= 50.0
    if case % 2 == 0 and n >= 8 * g:
        values[rng.integers(0, n, 1 + n // 300)] = np.nan
        values[rng.integers(0, n, 3)] = np.inf
        values[g:2 * g] = np.nan                      # nothing comparable
        values[2 * g:3 * g] = 0.0                     # nothing non-zero
        values[3 * g:4 * g] = -2.5                    # all equal
        values[4 * g:5 * g] = 0.0
        values[4 * g + 5] = 3.0                       # a single non-zero
        values[5 * g + g - 1] = np.nan                # a NaN that ends an fp32 scan
        values[6 * g:7 * g] = np.nan
        values[6 * g + 1] = 4.0                       # one comparable element among NaNs
    return values


@pytest.mark.parametrize("name", list(NAMES))
@pytest.mark.parametrize("g", (16, 32, 64))
@pytest.mark.parametrize("compact", (False, True))
def test_quantize_and_decode_bytes(hip, hip_device, name, g, compact):
    rng = np.random.default_rng(g + 7 * compact)
    for case, (bit, quant_type, topk, stochastic) in enumerate(policies()):
        n = g * int(rng.choice([1, 7, 70, 1031]))      # 1031 groups: tiles end inside the last block
        x_np = wire.from_f32(awkward_values(rng, n, g, case), name)
        x = from_numpy(x_np, name, hip_device)
        policy = dict(group_size=g, bit=bit, quant_type=quant_type, topk=topk, compact=compact)
        what = f"{name} g={g} {policy} stochastic={stochastic} n={n}"
        payload = torch.full((hip.general_payload_nbytes(n, x.dtype, g, bit, topk),), 0xA5, dtype=torch.uint8,
                             device=hip_device)
        assert hip.quant_general_into(x, payload, stochastic=stochastic, **policy), what
        want = general.quantize(x_np, name, g, bit, quant_type, topk, stochastic, compact)
        same(payload, want, "quantize " + what)
        old_np = wire.from_f32((rng.standard_normal(n) * 0.5).astype(np.float32), name)
        for op in ("none", "sum", "max", "min"):
            out = from_numpy(old_np, name, hip_device)
            assert hip.dequant_general_into(payload, out, reduce_op=op, **policy), what
            same(out, general.dequantize(want, n, name, g, bit, quant_type, topk, compact, op, old_np),
                 f"decode {op} " + what)


def test_randomized_policies_sizes_and_contents(hip, hip_device):
    """400 seeded draws over dtype, group, bit, code book, top-k, rounding seed, layout, size (1 to 30,000 groups)
    and content (scales 1e-8..1e3, NaN/Inf, many ties, many zeros): quantize bytes and one decode op each."""
    rng = np.random.default_rng(2718)
    for case in range(400):
        name = str(rng.choice(list(NAMES)))
        g, bit, topk = int(rng.choice([16, 32, 64])), int(rng.choice([4, 8])), int(rng.choice([0, 1, 2]))
        quant_type = "linear" if bit == 8 else str(rng.choice(general.QUANT_TYPES))
        stochastic = None if rng.random() < 0.4 else (int(rng.integers(0, 2 ** 63)), int(rng.integers(0, 2 ** 40)))
        compact = bool(rng.integers(0, 2))
        n = g * int(rng.choice([1, 3, 17, 64, 65, 255, 1024, 4097, 30000]))
        values = (rng.standard_normal(n) * 10.0 ** rng.integers(-8, 4)).astype(np.float32)
        content = int(rng.integers(0, 4))
        if content == 1:
            values[rng.integers(0, n, max(1, n // 50))] = np.nan
            values[rng.integers(0, n, 2)] = np.inf
        elif content == 2:
            values = np.round(values * 4) / 4
        elif content == 3:
            values[rng.integers(0, n, max(1, n // 3))] = 0
        x_np = wire.from_f32(values, name)
        x = from_numpy(x_np, name, hip_device)
        policy = dict(group_size=g, bit=bit, quant_type=quant_type, topk=topk, compact=compact)
        what = f"case {case}: {name} {policy} stochastic={stochastic} n={n} content={content}"
        payload = torch.empty(hip.general_payload_nbytes(n, x.dtype, g, bit, topk), dtype=torch.uint8, device=hip_device)
        assert hip.quant_general_into(x, payload, stochastic=stochastic, **policy), what
        want = general.quantize(x_np, name, g, bit, quant_type, topk, stochastic, compact)
        same(payload, want, "quantize " + what)
        op = str(rng.choice(["none", "sum", "max", "min"]))
        old_np = wire.from_f32(rng.standard_normal(n).astype(np.float32), name)
        out = from_numpy(old_np, name, hip_device)
        assert hip.dequant_general_into(payload, out, reduce_op=op, **policy), what
        same(out, general.dequantize(want, n, name, g, bit, quant_type, topk, compact, op, old_np), f"decode {op} " + what)


@pytest.mark.parametrize("name", list(NAMES))
def test_plain_policy_equals_the_pack_kernel_on_finite_input(hip, hip_device, name):
    n = 64 * 4000
    x = from_numpy(wire.from_f32((np.random.default_rng(3).standard_normal(n) * 0.02).astype(np.float32), name), name,
                   hip_device)
    for bit, compact in itertools.product((4, 8), (False, True)):
        fast = hip.quant_pack(x, group_size=64, compact=compact, bit=bit)
        payload = torch.empty_like(fast)
        assert hip.quant_general_into(x, payload, group_size=64, bit=bit, compact=compact)
        assert torch.equal(fast, payload)
        a, b = torch.empty_like(x), torch.empty_like(x)
        assert hip.dequant_into(fast, a, group_size=64, compact=compact, bit=bit)
        assert hip.dequant_general_into(fast, b, group_size=64, bit=bit, compact=compact)
        assert torch.equal(a.view(torch.int16 if name != "fp32" else torch.int32),
                           b.view(torch.int16 if name != "fp32" else torch.int32))


@pytest.mark.parametrize("name", list(NAMES))
@pytest.mark.parametrize("g", (16, 64))
def test_pack_entry_point_takes_the_maximum_as_the_reference_dispatch_does(hip, hip_device, name, g):
    """Whole groups without a residual: a NaN resets the running maximum (general kernels); with a residual or a
    ragged tail: NaNs are skipped (fused pack kernel).  Interior blocks and the edge block both see NaNs."""
    rng = np.random.default_rng(g)
    n = g * 3000
    values = awkward_values(rng, n, g, 0)
    values[rng.integers(0, n, 400)] = np.nan
    values[n - 3] = np.nan
    x_np = wire.from_f32(values, name)
    x = from_numpy(x_np, name, hip_device)
    r_np = wire.from_f32((rng.standard_normal(n) * 1e-3).astype(np.float32), name)
    r = from_numpy(r_np, name, hip_device)
    for bit, compact in itertools.product((8, 4), (True, False)):
        same(hip.quant_pack(x, group_size=g, compact=compact, bit=bit),
             general.quantize_pack(x_np, name, g, compact, None, bit), f"whole groups {bit} {compact}")
        assert not np.array_equal(general.quantize_pack(x_np, name, g, compact, None, bit),
                                  wire.quantize(x_np, name, g, compact, None, bit))
        same(hip.quant_pack(x, group_size=g, compact=compact, bit=bit, residual=r),
             wire.quantize(x_np, name, g, compact, r_np, bit), f"residual {bit} {compact}")
        same(hip.quant_pack(x[:n - 5], group_size=g, compact=compact, bit=bit),
             wire.quantize(x_np[:n - 5], name, g, compact, None, bit), f"ragged {bit} {compact}")
    # chunks: a chunk of whole groups follows the general kernels, the ragged last chunk the pack kernel
    world, total = 4, g * 1000 - 3
    shard = -(-total // world)
    assert shard == g * 250
    stride = hip.payload_nbytes(shard, x.dtype, g) + 8
    rows = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
    assert hip.bind_quant_pack_chunks(x[:total], rows, world, group_size=g)()
    for d in range(world):
        piece = x_np[d * shard:min(total, (d + 1) * shard)]
        want = general.quantize_pack(piece, name, g, True, None, 8)
        same(rows[d, :want.size], want, f"chunk {d}")


def test_contract_violations(hip, hip_device):
    x = torch.zeros(64 * 3, device=hip_device)
    payload = torch.empty(hip.general_payload_nbytes(x.numel(), x.dtype, 64, 8, 1), dtype=torch.uint8, device=hip_device)
    with pytest.raises(RuntimeError, match="multiple of group_size"):
        hip.quant_general_into(x[:100], payload, topk=1)
    with pytest.raises(RuntimeError, match="invalid quantized payload size"):
        hip.quant_general_into(x, payload[:-4], topk=1)
    with pytest.raises(RuntimeError, match="only supports 4-bit"):
        hip.quant_general_into(x, payload, quant_type="normal", bit=8)
    with pytest.raises(RuntimeError, match="topk must be"):
        hip.quant_general_into(x, payload, topk=3)
    empty = torch.empty(0, device=hip_device)
    assert hip.quant_general_into(empty, torch.empty(0, dtype=torch.uint8, device=hip_device), topk=2)


def test_philox_stream_matches_the_platform_library(hip, hip_device):
    """rocRAND's Philox4x32-10 device generator yields cuRAND's sequence for a (seed, subsequence, offset); the
    oracle's counter-mode stream, which the quantize kernel was checked against above, must yield the same words,
    and so must the stochastic codes of a payload rebuilt from the library's draws."""
    import ctypes
    from pathlib import Path

    path = Path(__file__).resolve().parent / "native" / "_build" / "librocrand_draws.so"
    assert path.exists(), "run __graft_entry__.build() first: it compiles tests/native/rocrand_draws.hip"
    helper = ctypes.CDLL(str(path))
    helper.rocrand_philox_draws.restype = ctypes.c_int
    helper.rocrand_philox_draws.argtypes = [ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64, ctypes.c_int,
                                            ctypes.c_void_p, ctypes.c_void_p]
    subsequences = np.array([0, 1, 2, 77, 2 ** 20 + 3, 2 ** 32 + 5, 2 ** 40], dtype=np.uint64)
    device_subsequences = torch.from_numpy(subsequences.view(np.int64)).to(hip_device)
    for seed, offset in ((0, 0), (42, 8), (7, 3), (0x0123456789ABCDEF, 2 ** 33 + 1), (2 ** 63 + 11, 6)):
        out = torch.zeros(len(subsequences) * 70, dtype=torch.int32, device=hip_device)
        stream = torch.cuda.current_stream(hip_device).cuda_stream
        assert helper.rocrand_philox_draws(seed, device_subsequences.data_ptr(), len(subsequences), offset, 70,
                                           out.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        library = out.cpu().numpy().view(np.uint32).reshape(len(subsequences), 70)
        assert np.array_equal(library, general.curand_draws(seed, subsequences, offset, 70)), (seed, offset)
    # end to end: the codes of group s are rint(fma(v, m, u - 0.5)) with u from the library's draws of subsequence s
    g, groups, seed, offset = 64, 96, 1234, 12
    x = torch.randn(g * groups, generator=torch.Generator(device=hip_device).manual_seed(1), device=hip_device)
    payload = torch.empty(hip.general_payload_nbytes(x.numel(), x.dtype, g, 8, 0), dtype=torch.uint8, device=hip_device)
    assert hip.quant_general_into(x, payload, group_size=g, stochastic=(seed, offset))
    rows = torch.arange(groups, dtype=torch.int64, device=hip_device)
    out = torch.zeros(groups * g, dtype=torch.int32, device=hip_device)
    assert helper.rocrand_philox_draws(seed, rows.data_ptr(), groups, offset, g, out.data_ptr(),
                                       torch.cuda.current_stream(hip_device).cuda_stream) == 0
    torch.cuda.synchronize()
    draws = out.cpu().numpy().view(np.uint32).reshape(groups, g)
    uniform = general.curand_uniform(draws)
    values = x.cpu().numpy().reshape(groups, g)
    multiplier = (np.float64(127.0) / np.abs(values).max(axis=1).astype(np.float64)).astype(np.float32)[:, None]
    noise = (uniform.astype(np.float64) - 0.5).astype(np.float32)
    want = np.clip(np.rint(wire.fma_f32(values, np.broadcast_to(multiplier, values.shape), noise)), -127, 127)
    codes, _ = general.split(to_numpy(payload), x.numel(), "fp32", g, 8, 0, False)
    assert np.array_equal(codes, want.astype(np.int8))


# --------------------------------------------------------------------------- #
# the extension module and the codec facade
# --------------------------------------------------------------------------- #
@pytest.fixture(scope="module")
def wire_status(hip_device):
    from lowbit_comm_amd.hip.loader import load_hip_extension

    status = load_hip_extension(wire_format="native")
    assert status.available, status.reason
    return status


@pytest.mark.parametrize("name", list(NAMES))
def test_module_runs_every_policy(wire_status, hip_device, name):
    module = wire_status.module
    kinds = {"linear": module.QuantType.Linear, "normal": module.QuantType.Normal, "uniform": module.QuantType.Uniform,
             "e3m0": module.QuantType.E3M0, "e2m1": module.QuantType.E2M1}
    dtype_member = {"fp32": module.DType.FP32, "fp16": module.DType.FP16, "bf16": module.DType.BF16}[name]
    rng = np.random.default_rng(17)
    n, g = 64 * 300, 64
    x_np = wire.from_f32(awkward_values(rng, n, g, 0), name)
    x = from_numpy(x_np, name, hip_device)
    for bit, quant_type, topk, stochastic in policies():
        for compact in (False, True):
            seeds = None
            if stochastic is not None:
                torch.cuda.manual_seed(stochastic[0])
                generator = torch.cuda.default_generators[hip_device.index or 0]
                generator.set_offset(4 * stochastic[1])
                seeds = (stochastic[0], 4 * stochastic[1])
            payload = module.quantize(x, g, topk, stochastic is not None, bit, kinds[quant_type], compact)
            same(payload, general.quantize(x_np, name, g, bit, quant_type, topk, seeds, compact),
                 f"{bit} {quant_type} {topk} {stochastic} {compact}")
            if seeds is not None:       # the generator moved on by numel draws, as philox_engine_inputs does
                assert torch.cuda.default_generators[hip_device.index or 0].get_offset() == seeds[1] + n
            out = module.dequantize(payload, g, topk, bit, module.ReduceOP.NONE, kinds[quant_type], dtype_member, compact)
            same(out, general.dequantize(to_numpy(payload), n, name, g, bit, quant_type, topk, compact))
            if topk or quant_type != "linear":
                assert module.inplace_quantize_pack(x, payload, None, g, topk, False, bit, kinds[quant_type], True) is False
    # the decode-and-add chain of two payloads with outliers
    pair = [module.quantize(x, g, 2, False, 8, kinds["linear"], True) for _ in range(2)]
    total = module.dequantize_reduce(pair, g, 2, 8, kinds["linear"], dtype_member, True)
    once = general.dequantize(to_numpy(pair[0]), n, name, g, 8, "linear", 2, True)
    same(total, general.dequantize(to_numpy(pair[1]), n, name, g, 8, "linear", 2, True, "sum", once))
    with pytest.raises(RuntimeError, match="multiple of group_size"):
        module.quantize(x[:100], g, 1, False, 8, kinds["linear"], True)
    with pytest.raises(RuntimeError, match="supports group_size"):
        module.quantize(x, g, 0, False, 8, kinds["normal"], True)


def test_facade_round_trip_with_outliers_and_code_book(wire_status, hip_device):
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.quantization import codec

    gen = torch.Generator(device=hip_device).manual_seed(8)
    x = torch.randn(64 * 500, generator=gen, device=hip_device, dtype=torch.float16)
    x[::97] *= 40
    for config in (CompressionConfig(topk=2), CompressionConfig(topk=1, compact=True),
                   CompressionConfig(bit=4, quant_type="normal", allow_experimental=True),
                   CompressionConfig(bit=4, quant_type="e2m1", topk=2, compact=True, allow_experimental=True)):
        payload = codec.quantize_tensor(x, config, extension_status=wire_status)
        restored = codec.dequantize_tensor(payload, tuple(x.shape), config, dtype="fp16", extension_status=wire_status)
        kind = config.quant_type
        want_bytes = general.quantize(to_numpy(x), "fp16", 64, config.bit, kind, config.topk, None, config.compact)
        buffer = payload.buffer if hasattr(payload, "buffer") else payload
        same(buffer, want_bytes, str(config))
        same(restored.reshape(-1), general.dequantize(want_bytes, x.numel(), "fp16", 64, config.bit, kind, config.topk,
                                                      config.compact), str(config))


# --------------------------------------------------------------------------- #
# the 100 MiB bucket: properties that need no oracle pass over the whole tensor
# --------------------------------------------------------------------------- #
FULL = 26_214_400


@pytest.mark.parametrize("name", ("fp32", "bf16"))
def test_full_bucket_top2_restores_outliers_and_bounds_the_rest(hip, hip_device, name):
    gen = torch.Generator(device=hip_device).manual_seed(1234)
    x = (torch.randn(FULL, generator=gen, device=hip_device) * 1e-3).to(NAMES[name])
    g = 64
    payload = torch.empty(hip.general_payload_nbytes(FULL, x.dtype, g, 8, 2), dtype=torch.uint8, device=hip_device)
    assert hip.quant_general_into(x, payload, group_size=g, topk=2, compact=True)
    out = torch.empty_like(x)
    assert hip.dequant_general_into(payload, out, group_size=g, topk=2, compact=True)
    rows, got = x.float().view(-1, g), out.float().view(-1, g)
    order = rows.abs().argsort(dim=1, descending=True)
    top = order[:, :2]
    assert torch.equal(rows.gather(1, top), got.gather(1, top))                 # outliers travel verbatim
    third = rows.abs().gather(1, order[:, 2:3])
    error = (rows - got).abs()
    slack = 2.0 ** (-8 if name == "bf16" else -23)
    assert bool((error <= third / 254 * 1.0001 + got.abs() * slack).all())
    # the oracle on the first and last 64 Ki elements
    for block in (slice(0, 65536), slice(FULL - 65536, FULL)):
        part = torch.empty(hip.general_payload_nbytes(65536, x.dtype, g, 8, 2), dtype=torch.uint8, device=hip_device)
        assert hip.quant_general_into(x[block].clone(), part, group_size=g, topk=2, compact=True)
        if block.start == 0:       # group indices (which fix the 16-bit scan start) match the full run only here
            same(payload[:part.numel()], to_numpy(part), "prefix of the full payload")
        same(part, general.quantize(to_numpy(x[block]), name, g, 8, "linear", 2, None, True), "block against the oracle")


def test_full_bucket_stochastic_rounding_is_unbiased_and_repeatable(hip, hip_device):
    gen = torch.Generator(device=hip_device).manual_seed(99)
    x = torch.randn(FULL, generator=gen, device=hip_device) * 1e-3
    g = 64
    payload = torch.empty(hip.general_payload_nbytes(FULL, x.dtype, g, 8, 0), dtype=torch.uint8, device=hip_device)
    again = torch.empty_like(payload)
    out = torch.empty_like(x)
    assert hip.quant_general_into(x, payload, group_size=g, stochastic=(2024, 1 << 20))
    assert hip.quant_general_into(x, again, group_size=g, stochastic=(2024, 1 << 20))
    assert torch.equal(payload, again)
    assert hip.quant_general_into(x, again, group_size=g, stochastic=(2024, (1 << 20) + 4 * FULL))
    assert not torch.equal(payload, again)
    assert hip.dequant_general_into(payload, out, group_size=g)
    step = x.view(-1, g).abs().amax(dim=1, keepdim=True) / 127
    error = ((out - x).view(-1, g) / step).double()
    assert float(error.abs().max()) <= 1.0 + 1e-3                               # one of the two neighbouring codes
    assert abs(float(error.mean())) < 5 * (1 / 6 / FULL) ** 0.5                 # variance of u(1-u) averaged is 1/6
    # nearest rounding on the same data has a smaller error but is no closer on average
    assert 0.15 < float((error ** 2).mean()) < 0.18
    same(payload[:64 * 1024], general.quantize(to_numpy(x[:65536]), "fp32", g, 8, "linear", 0, (2024, 1 << 20), False)[:64 * 1024],
         "codes of the first 1024 groups")


def test_more_than_2_to_the_31_elements_in_the_cuda_byte_format(hip, hip_device):
    """64-bit indexing in the pack, decode and general kernels: a 4.3 GB bf16 tensor of whole groups; windows at the
    start, across the 2^31 boundary and at the end are compared with the oracle.  Payload offsets pass 2^31 bytes
    too (2.2 GB interleaved, and the appended metadata of the general layout sits behind 2.1 GB of codes)."""
    g = 64
    n = (1 << 31) + g * 1024
    x = torch.empty(n, dtype=torch.bfloat16, device=hip_device)
    step = 1 << 28
    for i, a in enumerate(range(0, n, step)):
        b = min(a + step, n)
        gen = torch.Generator(device=hip_device).manual_seed(777 + i)
        x[a:b] = (torch.randn(b - a, generator=gen, device=hip_device) * 1e-3).to(torch.bfloat16)
    windows = [(0, 1 << 18), ((1 << 31) - g * 2048, (1 << 31) + g * 512), (n - g * 1024, n)]
    restored = torch.empty_like(x)

    def check(payload, per_group_bytes, make_window_payload, decode_window, what):
        for a, b in windows:
            first, groups = a // g, (b - a) // g
            # 16-bit scans start at an element that depends on the group index modulo 32: keep windows aligned to it
            assert first % 32 == 0
            piece = to_numpy(x[a:b])
            want = make_window_payload(piece)
            got = payload[first * per_group_bytes:(first + groups) * per_group_bytes]
            same(got, want, f"{what} payload window {a}")
            same(restored[a:b], decode_window(want, b - a), f"{what} decoded window {a}")

    # plain linear 8-bit, interleaved scales: the dedicated pack and decode kernels
    payload = hip.quant_pack(x, group_size=g, compact=True)
    assert hip.dequant_into(payload, restored, group_size=g, compact=True)
    check(payload, g + 2, lambda piece: general.quantize_pack(piece, "bf16", g, True, None, 8),
          lambda want, count: wire.dequantize(want, count, "bf16", g, True), "pack kernel")
    # the fused reduce of the payload with itself is exactly twice the single decode (a power-of-two scaling)
    doubled = torch.empty_like(x)
    assert hip.dequant_reduce_into([payload, payload], doubled, group_size=g, compact=True)
    for a, b in windows:
        assert torch.equal(doubled[a:b], restored[a:b] * 2), f"reduce window {a}"
    del payload, doubled
    # top-2 outliers with stochastic rounding, interleaved metadata: the general kernels
    policy = dict(group_size=g, bit=8, quant_type="linear", topk=2, compact=True)
    payload = torch.empty(hip.general_payload_nbytes(n, x.dtype, g, 8, 2), dtype=torch.uint8, device=hip_device)
    seeds = (99, 1 << 33)
    assert hip.quant_general_into(x, payload, stochastic=seeds, **policy)
    assert hip.dequant_general_into(payload, restored, **policy)

    per_group = g + 4 * 2
    for a, b in windows:
        first, groups = a // g, (b - a) // g
        want = general.quantize(to_numpy(x[a:b]), "bf16", g, 8, "linear", 2, seeds, True, first_group=first)
        same(payload[first * per_group:(first + groups) * per_group], want, f"general payload window {a}")
        same(restored[a:b], general.dequantize(want, b - a, "bf16", g, 8, "linear", 2, True), f"general decoded window {a}")


@pytest.mark.parametrize("quant_type", ("normal", "e2m1"))
def test_full_bucket_code_book_decode_is_the_nearest_entry(hip, hip_device, quant_type):
    gen = torch.Generator(device=hip_device).manual_seed(5)
    x = torch.randn(FULL, generator=gen, device=hip_device)
    g = 64
    payload = torch.empty(hip.general_payload_nbytes(FULL, x.dtype, g, 4, 0), dtype=torch.uint8, device=hip_device)
    out = torch.empty_like(x)
    assert hip.quant_general_into(x, payload, group_size=g, bit=4, quant_type=quant_type, compact=True)
    assert hip.dequant_general_into(payload, out, group_size=g, bit=4, quant_type=quant_type, compact=True)
    book = torch.from_numpy(general.CODE_BOOKS[quant_type][:15].copy()).to(hip_device)
    scale = x.view(-1, g).abs().amax(dim=1, keepdim=True)
    t = (x.view(-1, g) / scale)
    nearest = (t.unsqueeze(-1) - book).abs().amin(dim=-1)
    achieved = (out.view(-1, g) / scale - t).abs()
    assert bool((achieved <= nearest + 1e-6).all())


@pytest.mark.parametrize("name", ("fp16", "bf16"))
@pytest.mark.parametrize("quant_type", tuple(general.CODE_BOOKS))
def test_code_books_on_every_16_bit_quotient(hip, hip_device, name, quant_type):
    """Every finite 16-bit value v with |v| <= top, in groups whose first element is `top`, so that the scale is
    `top` and the quotients v / top sweep [-1, 1] through every step of the book: with top = 1 the quotient is the
    value itself, with top = 1.5 and 0.0791 it is a rounded division.  The kernels encode these with a table lookup;
    the bytes must be the oracle's."""
    g = 64
    bits = np.arange(0, 0x8000, dtype=np.uint16)
    for top in (1.0, 1.5, 0.0791):
        top_bits = wire.from_f32(np.array([top], dtype=np.float32), name)
        magnitudes = wire.to_f32(bits.view(top_bits.dtype), name)
        keep = bits[np.isfinite(magnitudes) & (magnitudes <= wire.to_f32(top_bits, name)[0])]
        both = np.concatenate([keep, keep | 0x8000]).astype(np.uint16)
        rows = -(-both.size // (g - 1))
        padded = np.zeros(rows * (g - 1), dtype=np.uint16)
        padded[:both.size] = both
        x_bits = np.empty((rows, g), dtype=np.uint16)
        x_bits[:, 0] = top_bits.view(np.uint16)[0]
        x_bits[:, 1:] = padded.reshape(rows, g - 1)
        x_np = x_bits.reshape(-1).view(top_bits.dtype)
        x = from_numpy(x_np, name, hip_device)
        n = x_np.size
        payload = torch.empty(hip.general_payload_nbytes(n, x.dtype, g, 4, 0), dtype=torch.uint8, device=hip_device)
        assert hip.quant_general_into(x, payload, group_size=g, bit=4, quant_type=quant_type, compact=True)
        same(payload, general.quantize(x_np, name, g, 4, quant_type, 0, None, True), f"{name} {quant_type} top={top}")


@pytest.mark.parametrize("seed", range(4))
def test_random_policies_sizes_and_values_against_the_oracle(hip, hip_device, seed):
    """A seeded random walk over what the systematic sweep fixes by hand: group counts from one to a few tens of
    thousands, magnitudes over twelve decades, NaN / Inf sprinkled in, many ties and zeros, every policy, both layouts,
    random Philox seeds and offsets (all four phases of a block), decode with every reduce op."""
    rng = np.random.default_rng(7100 + seed)
    for case in range(60):
        name = str(rng.choice(list(NAMES)))
        g = int(rng.choice([16, 32, 64]))
        bit = int(rng.choice([4, 8]))
        quant_type = "linear" if bit == 8 else str(rng.choice(general.QUANT_TYPES))
        topk = int(rng.choice([0, 1, 2]))
        stochastic = None if rng.random() < 0.4 else (int(rng.integers(0, 2**63)), int(rng.integers(0, 2**40)))
        compact = bool(rng.integers(0, 2))
        groups = int(rng.choice([1, 3, 17, 64, 65, 255, 1024, 4097, 20000]))
        n = g * groups
        values = (rng.standard_normal(n) * 10.0 ** rng.integers(-8, 4)).astype(np.float32)
        mode = int(rng.integers(0, 4))
        if mode == 1:
            values[rng.integers(0, n, max(1, n // 50))] = np.nan
            values[rng.integers(0, n, 2)] = np.inf
        elif mode == 2:
            values = np.round(values * 4) / 4           # many ties and zeros
        elif mode == 3:
            values[rng.integers(0, n, max(1, n // 3))] = 0
        what = (f"seed {seed} case {case}: {name} g={g} bit={bit} {quant_type} topk={topk} stochastic={stochastic} "
                f"compact={compact} groups={groups} mode={mode}")
        x_np = wire.from_f32(values, name)
        x = from_numpy(x_np, name, hip_device)
        payload = torch.empty(hip.general_payload_nbytes(n, x.dtype, g, bit, topk), dtype=torch.uint8, device=hip_device)
        policy = dict(group_size=g, bit=bit, quant_type=quant_type, topk=topk, compact=compact)
        hip.quant_general_into(x, payload, stochastic=stochastic, **policy)
        want = general.quantize(x_np, name, g, bit, quant_type, topk, stochastic, compact)
        assert to_numpy(payload).tobytes() == want.tobytes(), f"{what}: payload bytes"
        op = str(rng.choice(["none", "sum", "max", "min"]))
        old_np = wire.from_f32(rng.standard_normal(n).astype(np.float32), name)
        out = from_numpy(old_np, name, hip_device)
        hip.dequant_general_into(payload, out, reduce_op=op, **policy)
        decoded = general.dequantize(want, n, name, g, bit, quant_type, topk, compact, op, old_np)
        assert to_numpy(out).tobytes() == decoded.tobytes(), f"{what}: decoded values ({op})"
