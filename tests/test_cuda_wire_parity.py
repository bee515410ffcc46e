"""GPU parity of the CUDA-wire-format kernels against the CPU oracle (oracle/cuda_wire_np.py): payload bytes,
decoded values, fused reduce and error feedback, all bit-exact."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import cuda_wire_np as wire
from oracle import cuda_wire_scalar as wire_c

pytestmark = pytest.mark.gpu

NAMES = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


@pytest.fixture(scope="module")
def hip(hip_device):
    from lowbit_comm_amd.hip import cuda_wire

    return cuda_wire


@pytest.fixture(params=["cached", "stream"])
def access(request):
    from lowbit_comm_amd.hip import ops as hip_ops

    with hip_ops.access_mode(request.param):
        yield request.param


def to_numpy(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def from_numpy(a: np.ndarray, name: str, device) -> torch.Tensor:
    if name == "bf16":
        return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16).to(device)
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def make(n, name, seed, device, sigma=1.0, offset=0):
    rng = np.random.default_rng(seed)
    values = (rng.standard_normal(n + offset) * sigma).astype(np.float32)
    values[rng.integers(0, n + offset, size=max(1, n // 997))] *= 30.0        # outliers
    return from_numpy(wire.from_f32(values, name), name, device)[offset:]


def same(a: torch.Tensor, b: np.ndarray, what=""):
    got = to_numpy(a)
    assert got.dtype == b.dtype and got.shape == b.shape, (what, got.dtype, b.dtype, got.shape, b.shape)
    if got.tobytes() != b.tobytes():
        bad = np.flatnonzero(got.view(np.uint8 if got.dtype == np.uint8 else got.dtype) != b)
        raise AssertionError(f"{what}: {bad.size} of {b.size} differ, first at {bad[:5]}: {got[bad[:5]]} vs {b[bad[:5]]}")


# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("name", list(NAMES))
@pytest.mark.parametrize("compact", (True, False))
@pytest.mark.parametrize("g", (16, 32, 64))
@pytest.mark.parametrize("n", (1, 63, 64, 131, 8192, 70_001))
def test_quantize_bytes(hip, hip_device, access, name, compact, g, n):
    x = make(n, name, 100 + n + g, hip_device, sigma=10.0 ** ((n % 7) - 4))
    r = make(n, name, 200 + n + g, hip_device, sigma=1e-3)
    same(hip.quant_pack(x, group_size=g, compact=compact), wire.quantize(to_numpy(x), name, g, compact), "plain")
    same(hip.quant_pack(x, group_size=g, compact=compact, residual=r),
         wire.quantize(to_numpy(x), name, g, compact, residual=to_numpy(r)), "with residual")


@pytest.mark.parametrize("name", list(NAMES))
def test_quantize_unaligned_views_and_inputs_untouched(hip, hip_device, access, name):
    """tests/cuda/test_fused_quant_pack.py:98-121 in the reference: contiguous views that start off a 16-byte boundary."""
    n = 20_000
    x = make(n, name, 5, hip_device, offset=1)
    r = make(n, name, 6, hip_device, sigma=0.01, offset=3)
    assert x.data_ptr() % 16 != 0 and r.data_ptr() % 16 != 0
    x0, r0 = x.clone(), r.clone()
    store = torch.empty(hip.payload_nbytes(n, x.dtype) + 8, dtype=torch.uint8, device=hip_device)
    shift = 2 if name != "fp32" else 4
    payload = store[shift:shift + hip.payload_nbytes(n, x.dtype)]               # payload itself only element-aligned
    assert hip.quant_pack_into(x, payload, residual=r)
    same(payload, wire.quantize(to_numpy(x), name, 64, True, residual=to_numpy(r)))
    assert torch.equal(x, x0) and torch.equal(r, r0)
    out = torch.empty(n + 1, dtype=x.dtype, device=hip_device)[1:]
    assert hip.dequant_into(payload, out)
    same(out, wire.dequantize(to_numpy(payload), n, name))


def test_quantize_matches_reference_test_inputs(hip, hip_device):
    """The inputs of tests/cuda/test_fused_quant_pack.py:27-70 (linspace, group + 7 elements, with and without
    residual): the fused path must equal quantizing ``tensor + residual``."""
    for name, dtype in NAMES.items():
        for g in (16, 32, 64):
            tensor = torch.linspace(-3.0, 3.0, g + 7, device=hip_device, dtype=dtype)
            residual = torch.linspace(-0.2, 0.2, g + 7, device=hip_device, dtype=dtype)
            fused = hip.quant_pack(tensor, group_size=g, residual=residual)
            chained = hip.quant_pack(tensor + residual, group_size=g)
            assert fused.numel() == 2 * (g + tensor.element_size())
            assert torch.equal(fused, chained)
            same(fused, wire.quantize(to_numpy(tensor), name, g, True, residual=to_numpy(residual)))


def test_non_finite_and_tiny_groups(hip, hip_device):
    x = torch.ones(256, device=hip_device)
    x[3] = float("nan")
    x[70] = float("inf")
    x[128:192] = 1.0e-8
    x[192:] = 0.0
    same(hip.quant_pack(x), wire.quantize(to_numpy(x), "fp32"))
    h = x.to(torch.float16)
    same(hip.quant_pack(h), wire.quantize(to_numpy(h), "fp16"))
    assert hip.quant_pack(torch.empty(0, device=hip_device)).numel() == 0


# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("name", list(NAMES))
@pytest.mark.parametrize("compact", (True, False))
@pytest.mark.parametrize("g", (16, 64))
@pytest.mark.parametrize("op", ("none", "sum", "max", "min"))
def test_dequantize_and_reduce_ops(hip, hip_device, access, name, compact, g, op):
    for n in (77, 4096, 33_333):
        x = make(n, name, 300 + n, hip_device)
        payload = hip.quant_pack(x, group_size=g, compact=compact)
        base = make(n, name, 400 + n, hip_device, sigma=50.0 if op == "sum" else 1.0)
        out = base.clone()
        assert hip.dequant_into(payload, out, group_size=g, compact=compact, reduce_op=op)
        same(out, wire.dequantize(to_numpy(payload), n, name, g, compact, op, to_numpy(base)), f"{op} n={n}")


@pytest.mark.parametrize("name", ("fp16", "bf16"))
def test_sum_op_is_one_rounding(hip, hip_device, name):
    """out += decoded must round the exact sum once (native half add), not a float32 sum a second time."""
    n = 64 * 4000
    x = make(n, name, 9, hip_device, sigma=0.05)
    payload = hip.quant_pack(x)
    base = make(n, name, 10, hip_device, sigma=100.0)
    out = base.clone()
    assert hip.dequant_into(payload, out, reduce_op="sum")
    decoded = torch.empty_like(x)
    assert hip.dequant_into(payload, decoded)
    same(out, wire.dequantize(to_numpy(payload), n, name, reduce_op="sum", out=to_numpy(base)))
    same(out, wire_c.dequantize(to_numpy(payload), n, name, reduce_op="sum", out=to_numpy(base)))


# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("name", list(NAMES))
@pytest.mark.parametrize("compact", (True, False))
@pytest.mark.parametrize("world", (1, 2, 3, 8))
@pytest.mark.parametrize("fma", (True, False))
def test_fused_reduce_and_error_feedback(hip, hip_device, access, name, compact, world, fma):
    for n in (64, 64 * 129, 100_003):
        grads = [make(n, name, 500 + 10 * world + r, hip_device, sigma=10.0 ** (r % 3 - 2)) for r in range(world)]
        payloads = [hip.quant_pack(g_, compact=compact) for g_ in grads]
        host = [to_numpy(p) for p in payloads]
        inv = float(np.float32(1.0) / np.float32(world))
        out = torch.empty(n, dtype=NAMES[name], device=hip_device)
        assert hip.dequant_reduce_into(payloads, out, compact=compact, inv_divisor=inv, fused_multiply_add=fma)
        same(out, wire.reduce_payloads(host, n, name, 64, compact, inv, fma), f"reduce n={n}")
        prepared = make(n, name, 600 + world, hip_device)
        residual = torch.empty_like(prepared)
        assert hip.dequant_reduce_into(payloads, out, compact=compact, inv_divisor=inv, fused_multiply_add=fma,
                                       prepared=prepared, new_residual=residual)
        want_restored, want_residual = wire.reduce_mean_error_feedback(host, to_numpy(prepared), n, name, 64, compact,
                                                                       world, fma)
        same(out, want_restored, f"restored n={n}")
        same(residual, want_residual, f"residual n={n}")
        # in place: the residual buffer may be the prepared buffer
        alias = prepared.clone()
        assert hip.dequant_reduce_into(payloads, out, compact=compact, inv_divisor=inv, fused_multiply_add=fma,
                                       prepared=alias, new_residual=alias)
        same(alias, want_residual, f"aliased residual n={n}")


@pytest.mark.parametrize("name", ("fp16", "bf16"))
@pytest.mark.parametrize("world", (2, 3, 8))
def test_fused_reduce_of_interleaved_16_bit_payloads_at_any_2_byte_alignment(hip, hip_device, access, name, world):
    """Payloads of 66-byte groups are read through aligned 12-byte windows with the scales taken out of the windows;
    a payload may start at any 2-byte aligned address, and the blocks of the fast path reach the payload's last
    group when the element count is a multiple of theirs."""
    for n, lead in ((2048 * 5, 0), (2048 * 5, 2), (4096 * 3, 6), (2048 * 4 + 64 * 3, 2), (100_003, 10)):
        grads = [make(n, name, 900 + 10 * world + r, hip_device, sigma=10.0 ** (r % 3 - 2)) for r in range(world)]
        packed = [hip.quant_pack(g_, compact=True) for g_ in grads]
        holders = [torch.zeros(p.numel() + 32, dtype=torch.uint8, device=hip_device) for p in packed]
        payloads = []
        for holder, p in zip(holders, packed):
            holder[lead:lead + p.numel()].copy_(p)
            holder[lead + p.numel():].fill_(0xA5)              # whatever follows a payload must not matter
            payloads.append(holder[lead:lead + p.numel()])
        host = [to_numpy(p) for p in packed]
        inv = float(np.float32(1.0) / np.float32(world))
        out = torch.empty(n, dtype=NAMES[name], device=hip_device)
        assert hip.dequant_reduce_into(payloads, out, compact=True, inv_divisor=inv, fused_multiply_add=False)
        same(out, wire.reduce_payloads(host, n, name, 64, True, inv, False), f"reduce n={n} lead={lead}")
        prepared = make(n, name, 950 + world, hip_device)
        residual = torch.empty_like(prepared)
        assert hip.dequant_reduce_into(payloads, out, compact=True, inv_divisor=inv, prepared=prepared, new_residual=residual)
        want_restored, want_residual = wire.reduce_mean_error_feedback(host, to_numpy(prepared), n, name, 64, True, world, True)
        same(out, want_restored, f"restored n={n} lead={lead}")
        same(residual, want_residual, f"residual n={n} lead={lead}")


def test_reduce_rejections(hip, hip_device):
    x = make(640, "fp16", 1, hip_device)
    payload = hip.quant_pack(x)
    out = torch.empty_like(x)
    assert hip.dequant_reduce_into([payload] * 9, out) is False                      # more than 8 payloads
    p32 = hip.quant_pack(x, group_size=32)
    assert hip.dequant_reduce_into([p32], out, group_size=32) is False               # fused reduce is group-64 only
    with pytest.raises(RuntimeError):
        hip.dequant_reduce_into([], out)
    with pytest.raises(RuntimeError):
        hip.dequant_reduce_into([payload[:-2]], out)
    with pytest.raises(RuntimeError):
        hip.quant_pack_into(x, torch.empty(10, dtype=torch.uint8, device=hip_device))
    with pytest.raises(RuntimeError):
        hip.quant_pack_into(x, payload, residual=x.float())


# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("name", list(NAMES))
@pytest.mark.parametrize("compact", (True, False))
def test_chunked_quantize_and_decode(hip, hip_device, access, name, compact):
    world, n = 8, 1_000_003
    x = make(n, name, 77, hip_device)
    shard = -(-n // world)
    row = hip.payload_nbytes(shard, x.dtype)
    payloads = torch.zeros(world, row + 8, dtype=torch.uint8, device=hip_device)[:, :row]   # strided rows
    assert hip.bind_quant_pack_chunks(x, payloads, world, compact=compact)()
    xs = to_numpy(x)
    for d in range(world):
        piece = xs[d * shard:min(n, (d + 1) * shard)]
        padded = np.zeros(shard, dtype=piece.dtype)
        padded[:piece.size] = piece
        same(payloads[d], wire.quantize(padded, name, 64, compact), f"chunk {d}")
    out = torch.empty(n, dtype=x.dtype, device=hip_device)
    assert hip.bind_dequant_chunks(payloads, out, shard, compact=compact)()
    want = np.concatenate([wire.dequantize(to_numpy(payloads[d]), shard, name, 64, compact) for d in range(world)])[:n]
    same(out, want)


def test_full_bucket_against_scalar_c(hip, hip_device):
    """100 MiB fp32 bucket and 50 MiB bf16 bucket, W=8 shard reduce: bytes against the scalar C restatement."""
    n = 26_214_400
    for name in ("fp32", "bf16"):
        x = make(n, name, 2026, hip_device, sigma=1e-3)
        payload = hip.quant_pack(x)
        same(payload, wire_c.quantize(to_numpy(x), name))
        shard = n // 8
        payloads = [hip.quant_pack(make(shard, name, 3000 + r, hip_device, sigma=1e-3)) for r in range(8)]
        out = torch.empty(shard, dtype=NAMES[name], device=hip_device)
        assert hip.dequant_reduce_into(payloads, out, inv_divisor=0.125)
        same(out, wire_c.reduce_payloads([to_numpy(p) for p in payloads], shard, name, inv_divisor=0.125))
        back = torch.empty_like(x)
        assert hip.dequant_into(payload, back)
        err = (back.float() - x.float()).abs().reshape(-1, 64)
        bound = x.float().abs().reshape(-1, 64).amax(dim=1, keepdim=True) * (0.5 / 127 + 2.0 ** -7)
        assert bool((err <= bound).all())


def test_cross_format_round_trip_is_consistent(hip, hip_device):
    """A payload written here decodes, through the reader arithmetic, to within half a step of the input, and
    requantizing the decoded tensor reproduces the same codes (a fixed point), for every dtype."""
    for name in NAMES:
        x = make(64 * 500, name, 42, hip_device)
        payload = hip.quant_pack(x)
        back = torch.empty_like(x)
        assert hip.dequant_into(payload, back)
        again = hip.quant_pack(back)
        codes_a, _ = wire.split(to_numpy(payload), x.numel(), name)
        codes_b, _ = wire.split(to_numpy(again), x.numel(), name)
        assert np.abs(codes_a.astype(np.int16) - codes_b.astype(np.int16)).max() <= 1


# --------------------------------------------------------------------------- #
# the drop-in module (names and argument orders of the reference's pybind module) and the facade over it
# --------------------------------------------------------------------------- #
@pytest.fixture(scope="module")
def wire_status(hip_device):
    from lowbit_comm_amd.hip.loader import load_hip_extension

    status = load_hip_extension(wire_format="native")
    assert status.available, status.reason
    assert status.module.NATIVE_WIRE_FORMAT == "native"
    return status


def test_module_round_trip_like_the_reference_smoke_test(wire_status, hip_device):
    """tests/test_cuda_extension_smoke.py:15-34 upstream: 4096 fp16 randn, 8-bit linear, group 64, rel-L2 < 0.02."""
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.quantization.codec import dequantize_tensor, quantize_tensor

    tensor = make(4096, "fp16", 1, hip_device)
    config = CompressionConfig(bit=8, group_size=64, quant_type="linear")
    quantized = quantize_tensor(tensor, config, extension_status=wire_status)
    same(quantized, wire.quantize(to_numpy(tensor), "fp16", 64, config.compact))
    restored = dequantize_tensor(quantized, tensor.shape, config, dtype="fp16", extension_status=wire_status)
    assert restored.shape == tensor.shape and bool(torch.isfinite(restored).all())
    rel = float((tensor.float() - restored.float()).norm() / tensor.float().norm())
    assert rel < 0.02
    same(restored, wire.dequantize(to_numpy(quantized), 4096, "fp16", 64, config.compact))


@pytest.mark.parametrize("name", list(NAMES))
def test_module_fused_pack_equals_the_padded_chain(wire_status, hip_device, name):
    """tests/cuda/test_fused_quant_pack.py:27-70 upstream: uneven input, with and without residual; sizes from the
    facade's allocator; metadata as the reference records it."""
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.quantization.codec import allocate_quantized_buffer, inplace_quantize_pack, quantize_tensor

    for g in (16, 32, 64):
        config = CompressionConfig(bit=8, group_size=g, compact=True)
        tensor = torch.linspace(-3.0, 3.0, g + 7, device=hip_device, dtype=NAMES[name])
        for residual in (None, torch.linspace(-0.2, 0.2, g + 7, device=hip_device, dtype=NAMES[name])):
            reference_input = tensor if residual is None else tensor + residual
            chained = quantize_tensor(reference_input, config, extension_status=wire_status)
            output = allocate_quantized_buffer(tensor, config, dtype=name, wire_format="native")
            metadata = {}
            assert inplace_quantize_pack(tensor, output, residual, config, metadata, extension_status=wire_status)
            assert torch.equal(output, chained)
            assert metadata == {"original_numel": g + 7, "padded_numel": 2 * g, "padding_numel": g - 7,
                                "fused_quant_pack": True}


@pytest.mark.parametrize("name", list(NAMES))
def test_module_reduce_paths(wire_status, hip_device, name):
    """Fused path for whole groups; decode-and-add chain in the tensor dtype otherwise (pybind.cpp:39-56 upstream)."""
    module = wire_status.module
    linear, dtype_member = module.QuantType.Linear, {"fp32": module.DType.FP32, "fp16": module.DType.FP16,
                                                     "bf16": module.DType.BF16}[name]
    n = 64 * 50
    grads = [make(n, name, 900 + r, hip_device) for r in range(4)]
    payloads = [module.quantize(g_, 64, 0, False, 8, linear, True) for g_ in grads]
    host = [to_numpy(p) for p in payloads]
    fused = module.dequantize_reduce(payloads, 64, 0, 8, linear, dtype_member, True)
    same(fused, wire.reduce_payloads(host, n, name))
    out = torch.empty(n, dtype=NAMES[name], device=hip_device)
    assert module.inplace_dequantize_reduce_mean(payloads, out, 64, 0, 8, linear, True, 4)
    same(out, wire.reduce_payloads(host, n, name, inv_divisor=0.25))
    # nine payloads: no fused kernel, the chain adds in the tensor dtype
    nine = payloads + payloads + payloads[:1]
    assert module.inplace_dequantize_reduce_mean(nine, out, 64, 0, 8, linear, True, 9) is False
    module.inplace_dequantize_reduce(nine, out, 64, 0, 8, linear, True)
    want = wire.dequantize(host[0], n, name)
    for p in (host + host + host[:1])[1:]:
        want = wire.dequantize(p, n, name, reduce_op="sum", out=want)
    same(out, want)
    # group size 32: chain as well
    p32 = [module.quantize(g_, 32, 0, False, 8, linear, True) for g_ in grads[:2]]
    got = module.dequantize_reduce(p32, 32, 0, 8, linear, dtype_member, True)
    want = wire.dequantize(to_numpy(p32[1]), n, name, 32, reduce_op="sum", out=wire.dequantize(to_numpy(p32[0]), n, name, 32))
    same(got, want)


def test_module_error_feedback_paths(wire_status, hip_device):
    """tests/test_cuda_extension_smoke.py:37-100 upstream: residual update, fused mean + feedback, ragged prepared."""
    module = wire_status.module
    linear = module.QuantType.Linear
    prepared = make(4096, "fp32", 3, hip_device)
    restored = make(4096, "fp32", 4, hip_device)
    residual = torch.empty_like(prepared)
    module.inplace_error_feedback_update(prepared, restored, residual)
    assert torch.equal(residual, prepared - restored)

    n = 131                                                       # ragged: restored workspace is padded to 192
    grads = [make(n, "fp16", 20 + r, hip_device) for r in range(2)]
    payloads = [module.quantize(torch.cat((g_, g_.new_zeros(192 - n))), 64, 0, False, 8, linear, True) for g_ in grads]
    prepared = make(n, "fp16", 30, hip_device)
    residual = torch.empty_like(prepared)
    restored = module.dequantize_reduce_update_error_feedback(payloads, prepared, residual, 64, 0, 8, linear,
                                                              module.DType.FP16, True, 2)
    assert restored.numel() == 192
    want_restored, want_residual = wire.reduce_mean_error_feedback([to_numpy(p) for p in payloads], to_numpy(prepared),
                                                                   n, "fp16", divisor=2)
    same(restored[:n], want_restored)
    same(residual, want_residual)
    with pytest.raises(RuntimeError):
        module.inplace_dequantize_reduce_mean_update_error_feedback(payloads, prepared, restored, residual, 64, 0, 8,
                                                                    linear, True, 0)
    with pytest.raises(RuntimeError):
        module.quantize(prepared, 64, 2, False, 8, linear, True)          # the general policies need whole groups
    assert module.inplace_quantize_pack(prepared, payloads[0], None, 64, 1, False, 8, linear, True) is False


# --------------------------------------------------------------------------- #
# 4-bit codes
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("name", list(NAMES))
@pytest.mark.parametrize("compact", (True, False))
@pytest.mark.parametrize("g", (16, 32, 64))
@pytest.mark.parametrize("n", (1, 63, 131, 8192, 70_001))
def test_four_bit_quantize_and_decode(hip, hip_device, access, name, compact, g, n):
    x = make(n, name, 1100 + n + g, hip_device, sigma=10.0 ** ((n % 7) - 4))
    r = make(n, name, 1200 + n + g, hip_device, sigma=1e-3)
    payload = hip.quant_pack(x, group_size=g, compact=compact, bit=4)
    assert payload.numel() == hip.payload_nbytes(n, x.dtype, g, 4)
    same(payload, wire.quantize(to_numpy(x), name, g, compact, bit=4), "plain")
    same(hip.quant_pack(x, group_size=g, compact=compact, residual=r, bit=4),
         wire.quantize(to_numpy(x), name, g, compact, residual=to_numpy(r), bit=4), "with residual")
    base = make(n, name, 1300 + n, hip_device, sigma=5.0)
    for op in ("none", "sum", "max", "min"):
        out = base.clone()
        assert hip.dequant_into(payload, out, group_size=g, compact=compact, reduce_op=op, bit=4)
        same(out, wire.dequantize(to_numpy(payload), n, name, g, compact, op, to_numpy(base), bit=4), op)


def test_four_bit_full_bucket_and_chunks(hip, hip_device, access):
    n, world = 26_214_400, 8
    x = make(n, "bf16", 77, hip_device, sigma=1e-3)
    payload = hip.quant_pack(x, bit=4)
    same(payload, wire_c.quantize(to_numpy(x), "bf16", bit=4))
    back = torch.empty_like(x)
    assert hip.dequant_into(payload, back, bit=4)
    same(back, wire_c.dequantize(to_numpy(payload), n, "bf16", bit=4))
    shard = n // world
    row = hip.payload_nbytes(shard, x.dtype, 64, 4)
    rows = torch.empty(world, row, dtype=torch.uint8, device=hip_device)
    assert hip.bind_quant_pack_chunks(x, rows, world, bit=4)()
    xs = to_numpy(x)
    for d in (0, 3, 7):
        same(rows[d], wire_c.quantize(xs[d * shard:(d + 1) * shard], "bf16", bit=4), f"chunk {d}")
    out = torch.empty_like(x)
    assert hip.bind_dequant_chunks(rows, out, shard, bit=4)()
    same(out, np.concatenate([wire_c.dequantize(to_numpy(rows[d]), shard, "bf16", bit=4) for d in range(world)]))


def test_four_bit_through_the_module(wire_status, hip_device):
    """4-bit codes are experimental upstream (allow_experimental); quantize and decode run natively, reduces chain."""
    from lowbit_comm_amd.config import CompressionConfig
    from lowbit_comm_amd.quantization.codec import allocate_quantized_buffer, dequantize_tensor, quantize_tensor

    module = wire_status.module
    linear = module.QuantType.Linear
    config = CompressionConfig(bit=4, group_size=64, compact=True, allow_experimental=True)
    tensor = make(64 * 30 + 5, "fp16", 8, hip_device)
    buffer = allocate_quantized_buffer(tensor, config, dtype="fp16", wire_format="native")
    assert buffer.numel() == 31 * (32 + 2)
    quantize_tensor(tensor, config, extension_status=wire_status, output=buffer)
    same(buffer, wire.quantize(to_numpy(tensor), "fp16", 64, True, bit=4))
    restored = dequantize_tensor(buffer, tensor.shape, config, dtype="fp16", extension_status=wire_status)
    same(restored, wire.dequantize(to_numpy(buffer), tensor.numel(), "fp16", bit=4))
    grads = [make(64 * 20, "fp16", 40 + r, hip_device) for r in range(3)]
    payloads = [module.quantize(g_, 64, 0, False, 4, linear, True) for g_ in grads]
    out = torch.empty(64 * 20, dtype=torch.float16, device=hip_device)
    assert module.inplace_dequantize_reduce_mean(payloads, out, 64, 0, 4, linear, True, 3) is False   # no fused 4-bit reduce
    module.inplace_dequantize_reduce(payloads, out, 64, 0, 4, linear, True)
    want = wire.dequantize(to_numpy(payloads[0]), 64 * 20, "fp16", bit=4)
    for p in payloads[1:]:
        want = wire.dequantize(to_numpy(p), 64 * 20, "fp16", reduce_op="sum", out=want, bit=4)
    same(out, want)
