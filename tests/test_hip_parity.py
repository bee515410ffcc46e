"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on the same seeded inputs.

Bar: int8 codes, fp32 scales and packed bytes bit-exact; decode / reduce / residual outputs bit-exact
(the kernels use the oracle's accumulation order and no FMA contraction), which is stricter than the
stated rtol 1e-6 / atol 1e-7.
"""
import numpy as np
import pytest
import torch

from oracle import codec_np, codec_torch

pytestmark = pytest.mark.gpu

DTYPES = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


@pytest.fixture(scope="module", params=["cached", "stream", "auto"])
def ops(request, hip_device):
    """The tensor-level ops with every launch bound under one access mode (plain cached accesses, non-temporal
    loads, or the library's own rule) - results must not depend on it."""
    from lowbit_comm_amd.hip import ops as hip_ops

    with hip_ops.access_mode(request.param):
        yield hip_ops


def gradient_like(n, dtype, seed, device, sigma=1e-3, outliers=True):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(n, generator=gen) * sigma
    if outliers and n:
        mask = torch.rand(n, generator=gen) < 1e-3
        x = torch.where(mask, torch.randn(n, generator=gen) * 1e-1, x)
    return x.to(dtype).to(device)


def bits(t: torch.Tensor) -> torch.Tensor:
    t = t.detach().cpu().contiguous()
    return t.view(torch.int32) if t.dtype == torch.float32 else t.view(torch.int16)


def assert_same_bits(got: torch.Tensor, want: torch.Tensor, what: str):
    assert got.dtype == want.dtype, what
    assert got.shape == want.shape, what
    same = torch.equal(bits(got), bits(want))
    if not same:
        bad = (bits(got) != bits(want)).nonzero().flatten()
        i = int(bad[0])
        raise AssertionError(f"{what}: {bad.numel()} mismatches, first at {i}: got {got.flatten()[i].item()!r} "
                             f"want {want.flatten()[i].item()!r}")


# --------------------------------------------------------------------------- #
# quantize + pack
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("n", [1, 63, 64, 65, 4096, 4097, 16384 + 256 * 3 + 17, 1_000_003])
def test_quant_pack_bit_exact(ops, hip_device, dtype, n):
    x = gradient_like(n, DTYPES[dtype], 1000 + n, hip_device)
    codes, scales = ops.quant_pack(x, group_size=64)
    want_codes, want_scales = codec_torch.quantize(x.cpu(), 64)
    assert torch.equal(codes.cpu(), want_codes)
    assert_same_bits(scales, want_scales, "scales")


@pytest.mark.parametrize("g", [16, 32, 64])
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_quant_pack_group_sizes(ops, hip_device, g, dtype):
    n = 70_001
    x = gradient_like(n, DTYPES[dtype], 77 + g, hip_device)
    codes, scales = ops.quant_pack(x, group_size=g)
    want_codes, want_scales = codec_torch.quantize(x.cpu(), g)
    assert torch.equal(codes.cpu(), want_codes)
    assert_same_bits(scales, want_scales, "scales")


def test_quant_pack_config1_bucket(ops, hip_device):
    """25 MiB fp32 DDP bucket, N(0,1e-3) with 0.1% N(0,1e-1) outliers: full size against the oracle."""
    n = 6_553_600
    x = gradient_like(n, torch.float32, 1234, hip_device)
    codes, scales = ops.quant_pack(x)
    want_codes, want_scales = codec_torch.quantize(x.cpu(), 64)
    assert torch.equal(codes.cpu(), want_codes)
    assert_same_bits(scales, want_scales, "scales")
    restored = ops.dequant(codes, scales, n)
    assert_same_bits(restored, codec_torch.dequantize(want_codes, want_scales, n), "round trip")
    rel = float((x - restored).norm() / x.norm())
    assert rel < 0.02


def test_quant_pack_special_values(ops, hip_device):
    x = torch.zeros(64 * 8, dtype=torch.float32)
    x[0:9] = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, 126.5])   # exact ties, scale 1.0
    x[64] = 1e-3                                                                    # next group: one value
    x[128:131] = torch.tensor([6e-7, -3.1e-7, 1.0e-7])                              # eps-clamped scale
    x[192:256] = 1e-40                                                              # denormals
    x[192] = 8e-8
    x[256] = float("nan")
    x[257] = 1.0
    x[320] = float("inf")
    x[321] = 2.0
    x[384] = 3.4e38                                                                 # near FLT_MAX
    x[385] = -1.7e38
    # group 7 stays all zero
    codes, scales = ops.quant_pack(x.to(hip_device))
    want_codes, want_scales = codec_np.quantize(x.numpy(), 64)
    got_scales = scales.cpu().numpy()
    finite = np.isfinite(want_scales)
    assert np.array_equal(got_scales[finite].view(np.uint32), want_scales[finite].view(np.uint32))
    assert np.isnan(got_scales[4]) and np.isinf(got_scales[5])
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    assert codes[:9].tolist() == [127, 0, 2, 2, 0, -2, -2, 4, 126]
    assert int(scales[7].view(torch.int32)) == 0x34000000


def test_quant_pack_near_tie_quotients(ops, hip_device):
    """Values built so that value/scale lands on or next to k + 0.5 - where a reciprocal multiply goes wrong."""
    rng = np.random.default_rng(5)
    groups = 4096
    x = np.zeros((groups, 64), dtype=np.float32)
    peak = rng.uniform(1e-4, 1e-2, size=groups).astype(np.float32)
    x[:, 0] = peak
    scale = np.maximum(peak / np.float32(127.0), np.float32(2.0 ** -23))
    k = rng.integers(-126, 126, size=(groups, 63)).astype(np.float32)
    base = (k + np.float32(0.5)) * scale[:, None]
    ulps = rng.integers(-2, 3, size=(groups, 63)).astype(np.int32)
    x[:, 1:] = (base.view(np.int32) + ulps).view(np.float32)
    x = np.where(np.abs(x) <= peak[:, None], x, 0).astype(np.float32).reshape(-1)
    codes, scales = ops.quant_pack(torch.from_numpy(x).to(hip_device))
    want_codes, want_scales = codec_np.quantize(x, 64)
    assert np.array_equal(scales.cpu().numpy().view(np.uint32), want_scales.view(np.uint32))
    assert np.array_equal(codes.cpu().numpy(), want_codes)


def test_quant_pack_unaligned_views_and_untouched_input(ops, hip_device):
    base = gradient_like(20_000, torch.float32, 9, hip_device)
    view = base[3:3 + 12_345]          # 12-byte offset: not 16-byte aligned
    keep = base.clone()
    storage = torch.empty(ops.payload_nbytes(view.numel()) + 1, dtype=torch.uint8, device=hip_device)
    groups = ops.num_groups(view.numel(), 64)
    codes = torch.empty(groups * 64 + 1, dtype=torch.int8, device=hip_device)[1:]   # odd address
    scales = torch.empty(groups, dtype=torch.float32, device=hip_device)
    assert ops.quant_pack_into(view, codes, scales)
    want_codes, want_scales = codec_torch.quantize(view.cpu(), 64)
    assert torch.equal(codes.cpu(), want_codes)
    assert_same_bits(scales, want_scales, "scales")
    assert torch.equal(base, keep)
    del storage


def test_packed_payload_bytes_match_the_wire_format(ops, hip_device):
    n = 10_000
    x = gradient_like(n, torch.float32, 21, hip_device)
    payload = torch.empty(ops.payload_nbytes(n), dtype=torch.uint8, device=hip_device)
    assert ops.quant_pack_payload_into(x, payload)
    want = codec_torch.pack(*codec_torch.quantize(x.cpu(), 64))
    assert payload.numel() == 157 * 68
    assert torch.equal(payload.cpu(), want)
    assert np.array_equal(payload.cpu().numpy(), codec_np.pack(*codec_np.quantize(x.cpu().numpy(), 64)))


def test_quantize_is_idempotent_and_scale_equivariant_at_full_size(ops, hip_device):
    """Size-independent properties on a 100 MiB fp32 bucket (too large to run the oracle on comfortably)."""
    n = 26_214_400
    x = gradient_like(n, torch.float32, 31, hip_device, outliers=False)
    codes, scales = ops.quant_pack(x)
    codes8, scales8 = ops.quant_pack(x * 8.0)
    assert torch.equal(codes, codes8)
    assert torch.equal(scales * 8.0, scales8)
    decoded = ops.dequant(codes, scales, n)
    codes2, _ = ops.quant_pack(decoded)
    assert torch.equal(codes, codes2)
    peak = codes.view(-1, 64).abs().amax(dim=1)
    assert int(peak.min()) == 127 and int(peak.max()) == 127
    err = (x - decoded).abs().view(-1, 64)
    assert bool((err <= scales[:, None] * 0.50005).all())


def test_more_than_2_to_the_31_elements(ops, hip_device):
    """Indexing is 64-bit: a 4.3 GB bf16 tensor with a ragged tail; group-aligned windows at the start, across
    the 2^31 boundary and at the tail are compared with the oracle (quantization is local to a group)."""
    n = (1 << 31) + 64 * 1000 + 5
    x = torch.empty(n, dtype=torch.bfloat16, device=hip_device)
    step = 1 << 28
    for i, a in enumerate(range(0, n, step)):
        b = min(a + step, n)
        gen = torch.Generator(device=hip_device).manual_seed(4242 + i)
        x[a:b] = (torch.randn(b - a, generator=gen, device=hip_device) * 1e-3).to(torch.bfloat16)
    codes, scales = ops.quant_pack(x)
    assert codes.numel() == ops.num_groups(n, 64) * 64 and scales.numel() == ops.num_groups(n, 64)
    restored = ops.dequant(codes, scales, n, dtype=torch.bfloat16)
    windows = [(0, 1 << 20), ((1 << 31) - 64 * 2000, (1 << 31) + 64 * 500), (n - 64 * 3000 - 5, n)]
    for a, b in windows:
        assert a % 64 == 0
        w_codes, w_scales = codec_torch.quantize(x[a:b].cpu(), 64)
        padded = ops.num_groups(b - a, 64) * 64
        assert torch.equal(codes[a:a + padded].cpu(), w_codes), (a, b)
        assert_same_bits(scales[a // 64:a // 64 + padded // 64], w_scales, f"scales {a}")
        assert_same_bits(restored[a:b], codec_torch.dequantize(w_codes, w_scales, b - a, 64, "bf16"), f"restored {a}")
    del restored
    # W=2 reduce across the boundary: x + x decodes to exactly twice the single decode
    out = torch.empty(n, dtype=torch.float32, device=hip_device)
    assert ops.dequant_reduce_into([(codes, scales), (codes, scales)], out)
    a, b = windows[1]
    single = codec_torch.dequantize(codes[a:b].cpu(), scales[a // 64:b // 64].cpu(), b - a, 64, "fp32")
    assert_same_bits(out[a:b], single + single, "reduce across 2^31")
    assert_same_bits(out[n - 1000:], codec_torch.dequantize(codes[windows[2][0]:].cpu(), scales[windows[2][0] // 64:].cpu(),
                                                            n - windows[2][0], 64, "fp32")[-1000:] * 2, "reduce tail")


# --------------------------------------------------------------------------- #
# decode and fused dequant-reduce
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("out_dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("n", [1, 64, 100, 16_384, 200_003])
def test_dequant_bit_exact(ops, hip_device, out_dtype, n):
    x = gradient_like(n, torch.float32, 300 + n, hip_device)
    codes, scales = ops.quant_pack(x)
    got = ops.dequant(codes, scales, n, dtype=DTYPES[out_dtype])
    want = codec_torch.dequantize(codes.cpu(), scales.cpu(), n, 64, out_dtype)
    assert_same_bits(got, want, "decoded")


def test_fp16_decode_rounds_twice_like_the_reference(ops, hip_device):
    """code*scale is rounded to fp32 and then to fp16 (two roundings).  A fused multiply-convert that rounds
    once differs on rare (code, scale) pairs; this payload is made only of such pairs."""
    rng = np.random.default_rng(77)
    picked_codes, picked_scales = [], []
    while len(picked_codes) < 4096:
        c = rng.integers(-127, 128, size=1 << 20).astype(np.int8)
        s = (rng.uniform(1e-6, 1e-3, size=1 << 20)).astype(np.float32)
        exact = c.astype(np.float64) * s.astype(np.float64)           # exact: 8 + 24 significant bits
        once = exact.astype(np.float16)
        twice = (c.astype(np.float32) * s).astype(np.float16)
        differs = once != twice
        picked_codes.extend(c[differs].tolist())
        picked_scales.extend(s[differs].tolist())
    groups = 4096
    codes = np.zeros((groups, 64), dtype=np.int8)
    codes[:, 0] = picked_codes[:groups]
    codes[:, 37] = picked_codes[:groups]
    scales = np.array(picked_scales[:groups], dtype=np.float32)
    t_codes = torch.from_numpy(codes.reshape(-1)).to(hip_device)
    t_scales = torch.from_numpy(scales).to(hip_device)
    n = groups * 64
    want = codec_torch.dequantize(t_codes.cpu(), t_scales.cpu(), n, 64, "fp16")
    assert_same_bits(ops.dequant(t_codes, t_scales, n, dtype=torch.float16), want, "decode")
    out = torch.empty(n, dtype=torch.float16, device=hip_device)
    assert ops.dequant_reduce_into([(t_codes, t_scales)], out)
    assert_same_bits(out, want, "reduce W=1")
    # and through the fused error-feedback quantize: restored = fp16(code*scale) of the payload just made
    x = want.float().to(hip_device)
    c2 = torch.empty(n, dtype=torch.int8, device=hip_device)
    s2 = torch.empty(groups, dtype=torch.float32, device=hip_device)
    restored = torch.empty(n, dtype=torch.float16, device=hip_device)
    half_in = x.half()
    assert ops.quant_pack_into(half_in, c2, s2, restored=restored)
    w_codes, w_scales, w_restored, _ = codec_torch.ef_round_trip(half_in.cpu(), None, 64, "fp16")
    assert torch.equal(c2.cpu(), w_codes)
    assert_same_bits(restored, w_restored, "restored")


@pytest.mark.parametrize("op", ["sum", "max", "min"])
def test_dequant_with_reduce_op_combines_with_existing_output(ops, hip_device, op):
    n = 70_000
    x = gradient_like(n, torch.float32, 41, hip_device)
    codes, scales = ops.quant_pack(x)
    before = gradient_like(n, torch.float32, 42, hip_device)
    out = before.clone()
    assert ops.dequant_into(codes, scales, out, reduce_op=op)
    decoded = codec_torch.dequantize(codes.cpu(), scales.cpu(), n)
    want = {"sum": before.cpu() + decoded, "max": torch.maximum(before.cpu(), decoded),
            "min": torch.minimum(before.cpu(), decoded)}[op]
    assert_same_bits(out, want, op)


def make_payloads(ops, world, n, device, seed, g=64):
    payloads = []
    for r in range(world):
        payloads.append(ops.quant_pack(gradient_like(n, torch.float32, seed + r, device, outliers=False), group_size=g))
    return payloads


@pytest.mark.parametrize("world", [1, 2, 3, 5, 8])
@pytest.mark.parametrize("n", [64, 1000, 16_384 * 3 + 5])
def test_dequant_reduce_sum_bit_exact(ops, hip_device, world, n):
    payloads = make_payloads(ops, world, n, hip_device, 500)
    out = torch.empty(n, dtype=torch.float32, device=hip_device)
    assert ops.dequant_reduce_into(payloads, out)
    want = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in payloads], n, 64, "fp32", "sum")
    assert_same_bits(out, want, "reduced")


@pytest.mark.parametrize("world", [3, 8])
@pytest.mark.parametrize("out_dtype", ["fp32", "fp16", "bf16"])
def test_dequant_reduce_mean_and_16bit_accumulation(ops, hip_device, world, out_dtype):
    n = 50_001
    payloads = make_payloads(ops, world, n, hip_device, 600)
    out = torch.empty(n, dtype=DTYPES[out_dtype], device=hip_device)
    assert ops.dequant_reduce_into(payloads, out, divisor=world)
    want = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in payloads], n, 64, out_dtype, "mean")
    assert_same_bits(out, want, "mean")


@pytest.mark.parametrize("out_dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("divisor", [8.0, 2.0, 0.5, 1024.0, 2.0 ** -20, 2.0 ** 125, 2.0 ** 126, 2.0 ** -125, 3.0, 7.0, 1.5])
def test_mean_divides_exactly_for_every_kind_of_divisor(ops, hip_device, out_dtype, divisor):
    """Power-of-two divisors take a product with the reciprocal inside the kernel, the others a division: either
    way the result is the true quotient, also where it is subnormal, overflows or starts from an infinity."""
    n, g = 64 * 257, 64
    rng = np.random.default_rng(int(abs(np.log2(divisor)) * 10) + 3)
    # every decoded value stays finite in the output type, so no sum is inf - inf (the sign of a generated NaN is
    # the one thing a CPU and a GPU may differ in); sums still overflow to infinity and quotients go subnormal
    if out_dtype == "fp16":
        scale_pool = np.array([1e-9, 1e-7, 6e-5, 1e-3, 1.0, 100.0, 500.0], dtype=np.float32)
    else:
        scale_pool = np.array([2.0 ** -140, 1e-38, 2.0 ** -126, 3e-30, 1e-3, 1.0, 1e30, 2e36], dtype=np.float32)
    payloads = []
    for _ in range(2):
        codes = torch.from_numpy(rng.integers(-127, 128, n, dtype=np.int8)).to(hip_device)
        scales = torch.from_numpy(rng.choice(scale_pool, n // g)).to(hip_device)
        payloads.append((codes, scales))
    out = torch.empty(n, dtype=DTYPES[out_dtype], device=hip_device)
    assert ops.dequant_reduce_into(payloads, out, divisor=divisor)
    total = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in payloads], n, g, out_dtype, "sum")
    want = (total.float() / torch.tensor(divisor, dtype=torch.float32)).to(DTYPES[out_dtype])
    assert_same_bits(out, want, f"mean by {divisor}")


def test_dequant_reduce_order_follows_the_list(ops, hip_device):
    n = 64 * 2000
    payloads = make_payloads(ops, 8, n, hip_device, 700)
    fwd = torch.empty(n, dtype=torch.float32, device=hip_device)
    rev = torch.empty_like(fwd)
    assert ops.dequant_reduce_into(payloads, fwd)
    assert ops.dequant_reduce_into(payloads[::-1], rev)
    cpu = [(c.cpu(), s.cpu()) for c, s in payloads]
    assert_same_bits(fwd, codec_torch.reduce_payloads(cpu, n), "forward")
    assert_same_bits(rev, codec_torch.reduce_payloads(cpu[::-1], n), "reverse")
    assert not torch.equal(fwd, rev)


def test_dequant_reduce_config2_shard(ops, hip_device):
    """W=8 payloads of a 3,276,800-element shard (100 MiB fp32 bucket split 8 ways), fixed rank order."""
    n = 3_276_800
    payloads = make_payloads(ops, 8, n, hip_device, 1234)
    out = torch.empty(n, dtype=torch.float32, device=hip_device)
    assert ops.dequant_reduce_into(payloads, out)
    want = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in payloads], n)
    assert_same_bits(out, want, "shard")


def test_dequant_reduce_linearity_at_full_bucket_size(ops, hip_device):
    """All-gather-reduce shape (8 payloads x 26,214,400): the W-way sum equals decode-and-add one by one."""
    n = 26_214_400
    x = gradient_like(n, torch.float32, 55, hip_device, outliers=False)
    payloads = []
    for r in range(8):
        payloads.append(ops.quant_pack(torch.roll(x, 4099 * r) * (1.0 + 0.25 * r)))
    fused = torch.empty(n, dtype=torch.float32, device=hip_device)
    assert ops.dequant_reduce_into(payloads, fused)
    chained = torch.empty_like(fused)
    for r, (codes, scales) in enumerate(payloads):
        assert ops.dequant_into(codes, scales, chained, reduce_op="none" if r == 0 else "sum")
    assert torch.equal(fused, chained)


def test_dequant_reduce_with_error_feedback_update(ops, hip_device):
    n = 40_000
    world = 4
    payloads = make_payloads(ops, world, n, hip_device, 800)
    prepared = gradient_like(n, torch.float32, 801, hip_device)
    restored = torch.empty(n, dtype=torch.float32, device=hip_device)
    residual = torch.empty_like(restored)
    assert ops.dequant_reduce_into(payloads, restored, divisor=world, prepared=prepared, new_residual=residual)
    want = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in payloads], n, 64, "fp32", "mean")
    assert_same_bits(restored, want, "restored")
    assert_same_bits(residual, prepared.cpu() - want, "residual")


def test_more_than_eight_payloads_is_unsupported_not_an_error(ops, hip_device):
    payloads = make_payloads(ops, 9, 128, hip_device, 900)
    out = torch.empty(128, dtype=torch.float32, device=hip_device)
    assert ops.dequant_reduce_into(payloads, out) is False


def test_contract_violations_raise(ops, hip_device):
    x = gradient_like(128, torch.float32, 1, hip_device)
    codes, scales = ops.quant_pack(x)
    out = torch.empty(128, dtype=torch.float32, device=hip_device)
    with pytest.raises(RuntimeError, match="divisor must be > 0"):
        ops.dequant_reduce_into([(codes, scales)], out, divisor=0)
    with pytest.raises(RuntimeError, match="inputs must not be empty"):
        ops.dequant_reduce_into([], out)
    with pytest.raises(RuntimeError, match="invalid quantized payload size"):
        ops.quant_pack_into(x, codes[:64], scales)
    with pytest.raises(RuntimeError, match="must be a GPU tensor"):
        ops.quant_pack_into(x.cpu(), codes, scales)
    with pytest.raises(RuntimeError, match="must be contiguous"):
        ops.quant_pack_into(torch.empty(128, 2, device=hip_device)[:, 0], codes, scales)


def test_empty_input_is_a_no_op(ops, hip_device):
    x = torch.empty(0, dtype=torch.float32, device=hip_device)
    codes, scales = ops.quant_pack(x)
    assert codes.numel() == 0 and scales.numel() == 0


# --------------------------------------------------------------------------- #
# error feedback
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("grad_dtype,res_dtype,restored_dtype", [
    ("bf16", "fp32", "fp32"), ("bf16", "fp32", "bf16"), ("fp16", "fp32", "fp16"), ("fp32", "fp32", "fp32"),
    ("bf16", "bf16", "bf16"), ("bf16", None, "bf16"), ("fp32", None, "fp32"), ("fp16", "fp16", "fp32"),
])
@pytest.mark.parametrize("n", [2048 * 5, 30_011])
def test_ef_quant_pack_matches_the_processor_round_trip(ops, hip_device, grad_dtype, res_dtype, restored_dtype, n):
    grad = gradient_like(n, DTYPES[grad_dtype], 1100 + n, hip_device)
    residual = None if res_dtype is None else gradient_like(n, DTYPES[res_dtype], 1101, hip_device, sigma=1e-5,
                                                             outliers=False)
    p_dtype = grad.dtype if residual is None else ops.promote(grad.dtype, residual.dtype)
    n_dtype = ops.promote(p_dtype, DTYPES[restored_dtype])
    groups = ops.num_groups(n, 64)
    codes = torch.empty(groups * 64, dtype=torch.int8, device=hip_device)
    scales = torch.empty(groups, dtype=torch.float32, device=hip_device)
    restored = torch.empty(n, dtype=DTYPES[restored_dtype], device=hip_device)
    new_residual = torch.empty(n, dtype=n_dtype, device=hip_device)
    assert ops.quant_pack_into(grad, codes, scales, residual=residual, new_residual=new_residual, restored=restored)
    w_codes, w_scales, w_restored, w_residual = codec_torch.ef_round_trip(
        grad.cpu(), None if residual is None else residual.cpu(), 64, restored_dtype)
    assert torch.equal(codes.cpu(), w_codes)
    assert_same_bits(scales, w_scales, "scales")
    assert_same_bits(restored, w_restored, "restored")
    assert_same_bits(new_residual, w_residual, "residual")


def test_ef_in_place_residual_over_ten_steps_config3_shape_scaled(ops, hip_device):
    """Config 3 at 1/16 size (3,276,800 bf16 values), 10 steps, residual updated in place."""
    n = 3_276_800
    residual = gradient_like(n, torch.float32, 1234, hip_device, sigma=1e-5, outliers=False)
    cpu_residual = residual.cpu()
    groups = ops.num_groups(n, 64)
    codes = torch.empty(groups * 64, dtype=torch.int8, device=hip_device)
    scales = torch.empty(groups, dtype=torch.float32, device=hip_device)
    for step in range(10):
        grad = gradient_like(n, torch.bfloat16, 2000 + step, hip_device, outliers=False)
        assert ops.quant_pack_into(grad, codes, scales, residual=residual, new_residual=residual)
        w_codes, w_scales, _w_restored, cpu_residual = codec_torch.ef_round_trip(grad.cpu(), cpu_residual, 64, "fp32")
        assert torch.equal(codes.cpu(), w_codes), f"step {step}"
        assert_same_bits(scales, w_scales, f"scales step {step}")
        assert_same_bits(residual, cpu_residual, f"residual step {step}")


@pytest.mark.parametrize("p,t", [("fp32", "fp32"), ("fp32", "bf16"), ("bf16", "bf16"), ("fp16", "fp32")])
def test_standalone_ef_update(ops, hip_device, p, t):
    n = 33_333
    prepared = gradient_like(n, DTYPES[p], 1, hip_device)
    restored = gradient_like(n, DTYPES[t], 2, hip_device)
    residual = torch.empty(n, dtype=ops.promote(DTYPES[p], DTYPES[t]), device=hip_device)
    assert ops.ef_update_into(prepared, restored, residual)
    assert_same_bits(residual, prepared.cpu() - restored.cpu(), "residual")


# --------------------------------------------------------------------------- #
# chunked plan (reduce-scatter leg + requantize + all-gather leg)
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("n,world", [(64 * 8 * 100, 8), (64 * 9 + 30, 4), (1_000_003, 8), (5, 8)])
def test_chunked_quantize_restarts_groups_per_chunk(ops, hip_device, n, world):
    x = gradient_like(n, torch.float32, 1300 + n, hip_device)
    shard = -(-n // world)
    stride = (ops.payload_nbytes(shard) + 15) // 16 * 16
    payloads = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
    assert ops.quant_pack_chunks_into(x, payloads, world)
    want = codec_np.quantize_chunks(x.cpu().numpy(), world, 64)
    for d, (codes, scales) in enumerate(want):
        row = payloads[d, :ops.payload_nbytes(shard)].cpu().numpy()
        assert np.array_equal(row, codec_np.pack(codes, scales)), f"chunk {d}"


@pytest.mark.parametrize("grad_dtype,res_dtype", [("bf16", "fp32"), ("fp32", "fp32"), ("bf16", "bf16"), ("fp16", None)])
@pytest.mark.parametrize("n,world", [(64 * 8 * 64, 8), (100_003, 4)])
def test_chunked_quantize_with_fused_error_feedback(ops, hip_device, grad_dtype, res_dtype, n, world):
    """One launch: p = g + r, every destination chunk of p quantized on its own, r' = p - decode(q) in place."""
    grad = gradient_like(n, DTYPES[grad_dtype], 1400 + n, hip_device)
    residual = None if res_dtype is None else gradient_like(n, DTYPES[res_dtype], 1401, hip_device, sigma=1e-5,
                                                             outliers=False)
    keep = None if residual is None else residual.clone()
    p_dtype = grad.dtype if residual is None else ops.promote(grad.dtype, residual.dtype)
    new_residual = residual if (residual is not None and residual.dtype == ops.promote(p_dtype, torch.float32)) \
        else torch.empty(n, dtype=ops.promote(p_dtype, torch.float32), device=hip_device)
    shard = -(-n // world)
    nbytes = ops.payload_nbytes(shard)
    stride = (nbytes + 15) // 16 * 16
    payloads = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
    assert ops.quant_pack_chunks_into(grad, payloads, world, residual=residual, new_residual=new_residual)
    prepared = grad.cpu() if keep is None else grad.cpu() + keep.cpu()
    padded = torch.cat([prepared.float(), torch.zeros(shard * world - n)])
    want_residual = torch.empty(shard * world)
    for d in range(world):
        chunk = padded[d * shard:(d + 1) * shard].to(prepared.dtype)
        codes, scales = codec_torch.quantize(chunk, 64)
        assert torch.equal(payloads[d, :nbytes].cpu(), codec_torch.pack(codes, scales)), f"chunk {d}"
        want_residual[d * shard:(d + 1) * shard] = (chunk - codec_torch.dequantize(codes, scales, shard, 64, "fp32")).float()
    assert_same_bits(new_residual, want_residual[:n].to(new_residual.dtype), "residual")


def test_full_plan_config4_scaled(ops, hip_device):
    """Config 4 at 1/32 size: quantize 8 chunks per peer, reduce, requantize, decode all shards."""
    world, n = 8, 1_638_400 + 40          # ragged: shard = 204_805
    peers = [gradient_like(n, torch.float32, 1234 + r, hip_device, outliers=False) for r in range(world)]
    shard = -(-n // world)
    nbytes = ops.payload_nbytes(shard)
    stride = (nbytes + 15) // 16 * 16
    sent = []
    for x in peers:
        rows = torch.empty(world, stride, dtype=torch.uint8, device=hip_device)
        assert ops.quant_pack_chunks_into(x, rows, world)
        sent.append(rows)
    gathered = torch.empty(world, stride, dtype=torch.uint8, device=hip_device)
    shards = []
    for dest in range(world):
        received = [ops.split_payload(sent[src][dest, :nbytes], shard) for src in range(world)]
        out = torch.empty(shard, dtype=torch.float32, device=hip_device)
        assert ops.dequant_reduce_into(received, out)
        shards.append(out)
        assert ops.quant_pack_payload_into(out, gathered[dest, :nbytes])
    restored = torch.empty(n, dtype=torch.float32, device=hip_device)
    assert ops.dequant_chunks_into(gathered, restored, shard)
    want_shards, want_restored = codec_np.reduce_scatter_all_gather_plan([p.cpu().numpy() for p in peers], 64, "sum")
    for d in range(world):
        assert np.array_equal(shards[d].cpu().numpy().view(np.uint32), want_shards[d].view(np.uint32)), f"shard {d}"
    assert np.array_equal(restored.cpu().numpy().view(np.uint32), want_restored.view(np.uint32))


# --------------------------------------------------------------------------- #
# randomized sweep over shapes, dtypes, groups, alignments and payload counts
# --------------------------------------------------------------------------- #
def test_randomized_parity_sweep(ops, hip_device):
    """60 seeded cases by default; LBC_SWEEP_CASES / LBC_SWEEP_SEED lengthen or reseed the sweep."""
    import os

    rng = np.random.default_rng(int(os.environ.get("LBC_SWEEP_SEED", "20261125")))
    names = ["fp32", "fp16", "bf16"]
    for case in range(int(os.environ.get("LBC_SWEEP_CASES", "60"))):
        g = int(rng.choice([16, 32, 64]))
        n = int(rng.integers(1, 200_000))
        x_name = names[int(rng.integers(0, 3))]
        offset = int(rng.integers(0, 4))                     # element offset: exercises unaligned base pointers
        sigma = float(10.0 ** rng.uniform(-6, 2))
        base = gradient_like(n + offset, DTYPES[x_name], 5000 + case, hip_device, sigma=sigma)
        x = base[offset:]
        label = f"case {case}: n={n} g={g} {x_name} offset={offset} sigma={sigma:.3g}"
        # plain quantize + decode to a random dtype
        codes, scales = ops.quant_pack(x, group_size=g)
        w_codes, w_scales = codec_torch.quantize(x.cpu(), g)
        assert torch.equal(codes.cpu(), w_codes), label
        assert_same_bits(scales, w_scales, label)
        o_name = names[int(rng.integers(0, 3))]
        assert_same_bits(ops.dequant(codes, scales, n, group_size=g, dtype=DTYPES[o_name]),
                         codec_torch.dequantize(w_codes, w_scales, n, g, o_name), label + f" decode {o_name}")
        # fused error feedback with a residual of a supported dtype
        r_name = [None, "fp32", x_name][int(rng.integers(0, 3))]
        d_name = ["fp32", x_name][int(rng.integers(0, 2))]
        residual = None if r_name is None else gradient_like(n, DTYPES[r_name], 6000 + case, hip_device, sigma=sigma * 1e-2)
        p_dtype = x.dtype if residual is None else ops.promote(x.dtype, residual.dtype)
        new_residual = torch.empty(n, dtype=ops.promote(p_dtype, DTYPES[d_name]), device=hip_device)
        restored = torch.empty(n, dtype=DTYPES[d_name], device=hip_device)
        groups = ops.num_groups(n, g)
        c2 = torch.empty(groups * g, dtype=torch.int8, device=hip_device)
        s2 = torch.empty(groups, dtype=torch.float32, device=hip_device)
        assert ops.quant_pack_into(x, c2, s2, group_size=g, residual=residual, new_residual=new_residual,
                                   restored=restored), label
        e_codes, e_scales, e_restored, e_residual = codec_torch.ef_round_trip(
            x.cpu(), None if residual is None else residual.cpu(), g, d_name)
        assert torch.equal(c2.cpu(), e_codes), label + " ef codes"
        assert_same_bits(s2, e_scales, label + " ef scales")
        assert_same_bits(restored, e_restored, label + " ef restored")
        assert_same_bits(new_residual, e_residual, label + " ef residual")
        # fused reduce of W payloads of this shape
        world = int(rng.integers(1, 9))
        payloads = [(codes, scales)] + [ops.quant_pack(gradient_like(n, torch.float32, 7000 + 10 * case + r, hip_device,
                                                                     sigma=sigma), group_size=g) for r in range(world - 1)]
        mode = ["sum", "mean"][int(rng.integers(0, 2))]
        out = torch.empty(n, dtype=DTYPES[o_name], device=hip_device)
        assert ops.dequant_reduce_into(payloads, out, group_size=g, divisor=float(world) if mode == "mean" else 1.0), label
        want = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in payloads], n, g, o_name, mode)
        assert_same_bits(out, want, label + f" reduce W={world} {mode} {o_name}")


# --------------------------------------------------------------------------- #
# fused reduce + requantize
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("mid", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("world", (1, 2, 5, 8))
@pytest.mark.parametrize("mode", ("sum", "mean"))
def test_reduce_requantize_equals_the_two_steps_and_the_oracle(ops, hip_device, mid, world, mode):
    for g, n in ((64, 64 * 300), (64, 100_003), (32, 4099), (16, 1), (64, 2_000_000)):
        peers = [gradient_like(n, torch.float32, 9000 + 7 * world + r, hip_device, sigma=10.0 ** (r % 3 - 3))
                 for r in range(world)]
        payloads = [ops.quant_pack(p, group_size=g) for p in peers]
        groups = ops.num_groups(n, g)
        codes = torch.empty(groups * g, dtype=torch.int8, device=hip_device)
        scales = torch.empty(groups, dtype=torch.float32, device=hip_device)
        divisor = float(world) if mode == "mean" else 1.0
        assert ops.dequant_reduce_quant_into(payloads, codes, scales, n, group_size=g, divisor=divisor,
                                             mid_dtype=DTYPES[mid])
        # against the oracle: reduce in `mid`, then quantize
        reduced = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in payloads], n, g, mid, mode)
        want_codes, want_scales = codec_torch.quantize(reduced, g)
        assert torch.equal(codes.cpu(), want_codes), (mid, world, mode, g, n)
        assert_same_bits(scales, want_scales, f"{mid} W={world} {mode} g={g} n={n}")
        # against the two launches
        shard = torch.empty(n, dtype=DTYPES[mid], device=hip_device)
        assert ops.dequant_reduce_into(payloads, shard, group_size=g, divisor=divisor)
        two_codes, two_scales = ops.quant_pack(shard, group_size=g)
        assert torch.equal(codes, two_codes) and torch.equal(scales.view(torch.int32), two_scales.view(torch.int32))


def test_reduce_requantize_contract(ops, hip_device):
    x = gradient_like(640, torch.float32, 1, hip_device)
    payload = ops.quant_pack(x)
    codes = torch.empty(640, dtype=torch.int8, device=hip_device)
    scales = torch.empty(10, dtype=torch.float32, device=hip_device)
    assert ops.dequant_reduce_quant_into([payload] * 9, codes, scales, 640) is False
    with pytest.raises(RuntimeError):
        ops.dequant_reduce_quant_into([], codes, scales, 640)
    with pytest.raises(RuntimeError):
        ops.dequant_reduce_quant_into([payload], codes[:100], scales, 640)
    with pytest.raises(RuntimeError):
        ops.dequant_reduce_quant_into([payload], payload[0], scales, 640)          # output aliases an input
    # a peer whose tail-group scale is not finite must not leak into the zero padding
    n = 70
    a, b = ops.quant_pack(gradient_like(n, torch.float32, 2, hip_device)), ops.quant_pack(gradient_like(n, torch.float32, 3, hip_device))
    b[1][1] = float("inf")
    c2 = torch.empty(128, dtype=torch.int8, device=hip_device)
    s2 = torch.empty(2, dtype=torch.float32, device=hip_device)
    assert ops.dequant_reduce_quant_into([a, b], c2, s2, n)
    reduced = codec_torch.reduce_payloads([(a[0].cpu(), a[1].cpu()), (b[0].cpu(), b[1].cpu())], n, 64, "fp32", "sum")
    want_codes, want_scales = codec_torch.quantize(reduced, 64)
    assert torch.equal(c2.cpu(), want_codes) and torch.equal(c2[n:].cpu(), torch.zeros(128 - n, dtype=torch.int8))
    assert_same_bits(s2, want_scales, "non-finite tail")


# --------------------------------------------------------------------------- #
# quantize of one bucket and reduce of another bucket's shard in one launch
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("grad_dtype,with_residual,out_dtype", [
    ("bf16", True, "fp32"), ("bf16", True, "bf16"), ("fp16", True, "fp32"), ("fp32", True, "fp32"), ("fp32", False, "fp32"),
    ("bf16", False, "bf16"), ("bf16", False, "fp32"), ("fp16", False, "fp16"),
])
@pytest.mark.parametrize("world,payloads", [(8, 8), (4, 2), (2, 4), (8, 3), (4, 5), (2, 7), (8, 6), (4, 1)])
@pytest.mark.parametrize("n,reduce_n", [(64 * 8 * 640, 64 * 640), (64 * 8 * 64 * 3 + 64 * 8, 50_048), (64 * 8 * 30, 4096 * 3)])
def test_shared_launch_of_quantize_and_reduce_equals_the_two_launches_and_the_oracle(
        ops, hip_device, grad_dtype, with_residual, out_dtype, world, payloads, n, reduce_n):
    grad = gradient_like(n, DTYPES[grad_dtype], 3100 + n, hip_device)
    residual = gradient_like(n, torch.float32, 3101, hip_device, sigma=1e-5, outliers=False) if with_residual else None
    keep = None if residual is None else residual.clone()
    shard = -(-n // world)
    stride = (ops.payload_nbytes(shard) + 255) // 256 * 256
    rows = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
    peers = [ops.quant_pack(gradient_like(reduce_n, torch.float32, 3200 + r, hip_device)) for r in range(payloads)]
    out = torch.empty(reduce_n, dtype=DTYPES[out_dtype], device=hip_device)
    quant = ops.bind_quant_pack_chunks(grad, rows, world, residual=residual, new_residual=residual)
    reduce = ops.bind_dequant_reduce(peers, out, divisor=float(payloads))
    both = ops.bind_quant_chunks_and_reduce(quant, reduce)
    assert both() is True
    got_rows, got_out = rows.clone(), out.clone()
    got_residual = None if residual is None else residual.clone()
    # the two launches on the same inputs
    rows.zero_(); out.zero_()
    if residual is not None:
        residual.copy_(keep)
    assert quant() and reduce()
    assert torch.equal(got_rows, rows)
    assert_same_bits(got_out, out.cpu(), "reduced shard")
    if residual is not None:
        assert_same_bits(got_residual, residual.cpu(), "residual")
    # and the oracle
    prepared = grad.cpu() if keep is None else grad.cpu() + keep.cpu()
    nbytes = ops.payload_nbytes(shard)
    for d in range(world):
        chunk = prepared[d * shard:(d + 1) * shard]
        if chunk.numel() < shard:
            chunk = torch.cat([chunk, torch.zeros(shard - chunk.numel(), dtype=chunk.dtype)])
        assert torch.equal(got_rows[d, :nbytes].cpu(), codec_torch.pack(*codec_torch.quantize(chunk, 64))), f"chunk {d}"
    want = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in peers], reduce_n, 64, out_dtype, "mean")
    assert_same_bits(got_out, want, "reduced shard against the oracle")


@pytest.mark.parametrize("grad_dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("n", [64 * 8 * 640, 64 * 8 * 64 * 3 + 64 * 8])
def test_shared_launch_with_a_16_bit_bucket_that_starts_a_residual_writes_an_fp32_residual(ops, hip_device, grad_dtype, n):
    """A 16-bit bucket without a residual whose new residual is asked for: `restored` is rounded to fp32, so the new
    residual is an fp32 tensor and the quantize half is the four-elements-per-lane instantiation - the shared launch
    has to run that one, not the pure 16-bit one."""
    world, reduce_n = 8, 64 * 640
    grad = gradient_like(n, DTYPES[grad_dtype], 3300 + n, hip_device)
    shard = -(-n // world)
    stride = (ops.payload_nbytes(shard) + 255) // 256 * 256
    rows = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
    guard = 4096
    arena = torch.full((n + 2 * guard,), 7.0, dtype=torch.float32, device=hip_device)     # catches a write past either end
    new_residual = arena[guard:guard + n]
    peers = [ops.quant_pack(gradient_like(reduce_n, torch.float32, 3400 + r, hip_device)) for r in range(world)]
    out = torch.empty(reduce_n, dtype=torch.float32, device=hip_device)
    quant = ops.bind_quant_pack_chunks(grad, rows, world, new_residual=new_residual)
    reduce = ops.bind_dequant_reduce(peers, out, divisor=float(world))
    assert ops.bind_quant_chunks_and_reduce(quant, reduce)() is True
    got_rows, got_out, got_residual = rows.clone(), out.clone(), new_residual.clone()
    assert torch.equal(arena[:guard].cpu(), torch.full((guard,), 7.0)) and torch.equal(arena[guard + n:].cpu(), torch.full((guard,), 7.0))
    rows.zero_(); out.zero_(); new_residual.zero_()
    assert quant() and reduce()
    assert torch.equal(got_rows, rows)
    assert_same_bits(got_out, out.cpu(), "reduced shard")
    assert_same_bits(got_residual, new_residual.cpu(), "new residual against the separate launch")
    nbytes = ops.payload_nbytes(shard)
    for d in range(world):
        chunk = grad.cpu()[d * shard:(d + 1) * shard]
        w_codes, w_scales, _w_restored, w_residual = codec_torch.ef_round_trip(chunk, None, 64, "fp32")
        assert torch.equal(got_rows[d, :nbytes].cpu(), codec_torch.pack(w_codes, w_scales)), f"chunk {d}"
        assert w_residual.dtype == torch.float32
        assert_same_bits(got_residual[d * shard:(d + 1) * shard], w_residual, f"new residual of chunk {d} against the oracle")


# --------------------------------------------------------------------------- #
# the sum of bucket and residual as an output of the quantize
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("grad_dtype,res_dtype,restored_dtype", [
    ("bf16", "fp32", "fp32"), ("bf16", "fp32", "bf16"), ("fp16", "fp32", "fp16"), ("fp32", "fp32", "fp32"),
    ("bf16", "bf16", "bf16"), ("bf16", None, "bf16"), ("fp32", None, "fp32"), ("fp16", "fp16", "fp32"),
])
@pytest.mark.parametrize("n", [2048 * 5, 30_011])
@pytest.mark.parametrize("with_feedback_outputs", [False, True])
def test_quantize_also_writes_prepared(ops, hip_device, grad_dtype, res_dtype, restored_dtype, n, with_feedback_outputs):
    """``prepared_out = bucket + residual`` in the torch promotion of their types - what
    ``ErrorFeedbackState.compensate`` returns (ccdl_comm/quantization/error_feedback.py:27-36) - from the launch that
    quantizes it; payload and the other outputs are those of the call without it."""
    grad = gradient_like(n, DTYPES[grad_dtype], 1100 + n, hip_device)
    residual = None if res_dtype is None else gradient_like(n, DTYPES[res_dtype], 1101, hip_device, sigma=1e-5,
                                                             outliers=False)
    p_dtype = grad.dtype if residual is None else ops.promote(grad.dtype, residual.dtype)
    groups = ops.num_groups(n, 64)
    codes = torch.empty(groups * 64, dtype=torch.int8, device=hip_device)
    scales = torch.empty(groups, dtype=torch.float32, device=hip_device)
    prepared = torch.full((n + 64,), 3.0, dtype=p_dtype, device=hip_device)
    restored = new_residual = None
    if with_feedback_outputs:
        restored = torch.empty(n, dtype=DTYPES[restored_dtype], device=hip_device)
        new_residual = torch.empty(n, dtype=ops.promote(p_dtype, DTYPES[restored_dtype]), device=hip_device)
    assert ops.quant_pack_into(grad, codes, scales, residual=residual, new_residual=new_residual, restored=restored,
                               restored_dtype=DTYPES[restored_dtype], prepared_out=prepared)
    want_prepared = grad.cpu() if residual is None else grad.cpu() + residual.cpu()
    assert want_prepared.dtype == p_dtype
    assert_same_bits(prepared[:n], want_prepared, "prepared")
    assert torch.equal(prepared[n:].cpu(), torch.full((64,), 3.0, dtype=p_dtype)), "written past the end"
    w_codes, w_scales, w_restored, w_residual = codec_torch.ef_round_trip(
        grad.cpu(), None if residual is None else residual.cpu(), 64, restored_dtype)
    assert torch.equal(codes.cpu(), w_codes)
    assert_same_bits(scales, w_scales, "scales")
    if with_feedback_outputs:
        assert_same_bits(restored, w_restored, "restored")
        assert_same_bits(new_residual, w_residual, "residual")


def test_quantize_chunks_also_write_prepared_and_refuse_a_wrong_type(ops, hip_device):
    world, n = 8, 64 * 8 * 100 + 8 * 5
    grad = gradient_like(n, torch.bfloat16, 1200, hip_device)
    residual = gradient_like(n, torch.float32, 1201, hip_device, sigma=1e-5, outliers=False)
    shard = -(-n // world)
    rows = torch.zeros(world, (ops.payload_nbytes(shard) + 255) // 256 * 256, dtype=torch.uint8, device=hip_device)
    plain = rows.clone()
    prepared = torch.empty(n, dtype=torch.float32, device=hip_device)
    assert ops.quant_pack_chunks_into(grad, rows, world, residual=residual, prepared_out=prepared)
    assert ops.quant_pack_chunks_into(grad, plain, world, residual=residual)
    assert torch.equal(rows, plain)
    assert_same_bits(prepared, grad.cpu() + residual.cpu(), "prepared")
    with pytest.raises(RuntimeError, match="prepared_out must have dtype"):
        ops.quant_pack_chunks_into(grad, rows, world, residual=residual, prepared_out=prepared.to(torch.bfloat16))
    with pytest.raises(RuntimeError, match="alias"):
        ops.quant_pack_chunks_into(grad.float(), rows, world, residual=residual, prepared_out=residual)


# --------------------------------------------------------------------------- #
# three stages of a bucket stream in one launch
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype,with_residual,track_residual", [
    ("bf16", True, True), ("fp16", True, True), ("fp32", True, True), ("fp32", False, False), ("bf16", False, False),
    ("fp16", False, False), ("bf16", False, True),
])
@pytest.mark.parametrize("world", [8, 4, 2, 3, 5, 6, 7, 1])
@pytest.mark.parametrize("stages", ["qrd", "qr", "qd", "rd", "q", "r", "d"])
@pytest.mark.parametrize("n", [64 * 8 * 640, 64 * 8 * 64 * 3 + 64 * 8 * 5])
def test_pipeline_step_equals_its_three_launches_and_the_oracle(ops, hip_device, dtype, with_residual, track_residual,
                                                                world, stages, n):
    """Quantize of bucket k, reduce + requantize for bucket k-1, decode of bucket k-2 in one grid: every output equal to
    the separate launches' and to the oracle's."""
    kind = DTYPES[dtype]
    n -= n % (64 * world)                 # shard boundaries on whole groups: the shared grid wants them 16-byte aligned
    shard = -(-n // world)
    nbytes = ops.payload_nbytes(shard)
    stride = (nbytes + 255) // 256 * 256
    grad = gradient_like(n, kind, 5100 + n, hip_device)
    residual = gradient_like(n, torch.float32, 5101, hip_device, sigma=1e-5, outliers=False) if with_residual else None
    new_residual = residual if with_residual else (torch.zeros(n, dtype=torch.float32, device=hip_device) if track_residual else None)
    keep = None if residual is None else residual.clone()
    send = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
    received = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
    for r in range(world):
        ops.quant_pack_payload_into(gradient_like(shard, kind, 5200 + r, hip_device), received[r, :nbytes])
    mine = torch.zeros(nbytes, dtype=torch.uint8, device=hip_device)
    gathered = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
    for r in range(world):
        ops.quant_pack_payload_into(gradient_like(shard, kind, 5300 + r, hip_device), gathered[r, :nbytes])
    decoded = torch.zeros(n, dtype=kind, device=hip_device)
    pairs = [ops.split_payload(received[r, :nbytes], shard) for r in range(world)]
    quant = ops.bind_quant_pack_chunks(grad, send, world, residual=residual, new_residual=new_residual)
    reduce = ops.bind_dequant_reduce_quant(pairs, *ops.split_payload(mine, shard), shard, divisor=float(world), mid_dtype=kind)
    decode = ops.bind_dequant_chunks(gathered, decoded, shard)
    step = ops.bind_bucket_pipeline_step(quant if "q" in stages else None, reduce if "r" in stages else None,
                                         decode if "d" in stages else None)
    assert step() is True
    got = [t.clone() for t in (send, mine, decoded)] + [None if new_residual is None else new_residual.clone()]
    for t in (send, mine, decoded):
        t.zero_()
    if residual is not None:
        residual.copy_(keep)
    elif new_residual is not None:
        new_residual.zero_()
    if "q" in stages:
        assert quant()
    if "r" in stages:
        assert reduce()
    if "d" in stages:
        assert decode()
    assert torch.equal(got[0], send), "payload rows"
    assert torch.equal(got[1], mine), "requantized shard payload"
    assert_same_bits(got[2], decoded.cpu(), "decoded bucket")
    if new_residual is not None:
        assert_same_bits(got[3], new_residual.cpu(), "residual")
    if "q" in stages:
        prepared = grad.cpu() if keep is None else grad.cpu() + keep.cpu()
        for d in range(world):
            chunk = prepared[d * shard:(d + 1) * shard]
            if chunk.numel() < shard:
                chunk = torch.cat([chunk, torch.zeros(shard - chunk.numel(), dtype=chunk.dtype)])
            assert torch.equal(got[0][d, :nbytes].cpu(), codec_torch.pack(*codec_torch.quantize(chunk, 64))), f"chunk {d}"
    if "r" in stages:
        reduced = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in pairs], shard, 64, dtype, "mean")
        assert torch.equal(got[1].cpu(), codec_torch.pack(*codec_torch.quantize(reduced, 64))), "reduce + requantize"
    if "d" in stages:
        for d in range(world):
            codes, scales = ops.split_payload(gathered[d, :nbytes], shard)
            want = codec_torch.dequantize(codes.cpu(), scales.cpu(), shard, 64, dtype)
            stop = min(n, (d + 1) * shard)
            assert_same_bits(got[2][d * shard:stop], want[:stop - d * shard], f"decoded shard {d}")


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_shared_grids_equal_their_separate_launches(ops, hip_device, seed):
    """Random bucket sizes, ranks, payload counts, types and stage subsets through both shared-grid entry points: every
    byte they write equals what the separate launches write.  (A stage's place in the grid - its row and its position
    in the row - comes out of a division by a run-time stride; sizes that are no round numbers walk that arithmetic.)"""
    rng = np.random.default_rng(8800 + seed)
    merged = 0
    for case in range(40):
        dtype = str(rng.choice(["fp32", "bf16", "fp16"]))
        kind = DTYPES[dtype]
        world = int(rng.integers(1, 9))
        n = 64 * world * int(rng.choice([rng.integers(1, 40), rng.integers(40, 3000)]))
        shard = n // world
        with_residual = bool(rng.integers(0, 2))
        what = f"seed {seed} case {case}: {dtype} n {n} world {world} residual {with_residual}"
        nbytes = ops.payload_nbytes(shard)
        stride = (nbytes + 255) // 256 * 256
        grad = gradient_like(n, kind, 8900 + 50 * seed + case, hip_device)
        residual = gradient_like(n, torch.float32, 8901 + case, hip_device, sigma=1e-5, outliers=False) if with_residual else None
        keep = None if residual is None else residual.clone()
        send = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
        quant = ops.bind_quant_pack_chunks(grad, send, world, residual=residual, new_residual=residual)

        def restore():
            send.zero_()
            if residual is not None:
                residual.copy_(keep)

        # the two-stage entry point: quantize + reduce of `payloads` payloads of another length
        payloads = int(rng.integers(1, 9))
        reduce_n = 64 * int(rng.integers(1, 1200)) + int(rng.choice([0, 0, 17]))
        peers = [ops.quant_pack(gradient_like(reduce_n, torch.float32, 9000 + r, hip_device)) for r in range(payloads)]
        out = torch.zeros(reduce_n, dtype=kind if rng.integers(0, 2) else torch.float32, device=hip_device)
        reduce = ops.bind_dequant_reduce(peers, out, divisor=float(payloads))
        if ops.bind_quant_chunks_and_reduce(quant, reduce)():
            merged += 1
            got = (send.clone(), out.clone(), None if residual is None else residual.clone())
            restore(); out.zero_()
            assert quant() and reduce(), what
            assert torch.equal(got[0], send) and torch.equal(got[1].view(torch.uint8), out.view(torch.uint8)), what
            assert residual is None or torch.equal(got[2].view(torch.uint8), residual.view(torch.uint8)), what
        restore()

        # the three-stage entry point on a random subset of its stages
        received = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
        gathered = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
        for r in range(world):
            ops.quant_pack_payload_into(gradient_like(shard, kind, 9100 + r, hip_device), received[r, :nbytes])
            ops.quant_pack_payload_into(gradient_like(shard, kind, 9200 + r, hip_device), gathered[r, :nbytes])
        mine = torch.zeros(nbytes, dtype=torch.uint8, device=hip_device)
        decoded = torch.zeros(n, dtype=kind, device=hip_device)
        pairs = [ops.split_payload(received[r, :nbytes], shard) for r in range(world)]
        requant = ops.bind_dequant_reduce_quant(pairs, *ops.split_payload(mine, shard), shard, divisor=float(world), mid_dtype=kind)
        decode = ops.bind_dequant_chunks(gathered, decoded, shard)
        stages = str(rng.choice(["qrd", "qr", "qd", "rd"]))
        step = ops.bind_bucket_pipeline_step(quant if "q" in stages else None, requant if "r" in stages else None,
                                             decode if "d" in stages else None)
        if step():
            merged += 1
            got = (send.clone(), mine.clone(), decoded.clone(), None if residual is None else residual.clone())
            restore(); mine.zero_(); decoded.zero_()
            for name, launch in (("q", quant), ("r", requant), ("d", decode)):
                if name in stages:
                    assert launch(), what
            assert torch.equal(got[0], send) and torch.equal(got[1], mine), f"{what} stages {stages}"
            assert torch.equal(got[2].view(torch.uint8), decoded.view(torch.uint8)), f"{what} stages {stages}"
            assert residual is None or torch.equal(got[3].view(torch.uint8), residual.view(torch.uint8)), f"{what} stages {stages}"
    assert merged >= 40, "most of these combinations have a shared grid"


def test_pipeline_step_without_a_shared_grid_says_so(ops, hip_device):
    """Another group size than 64, or operands that are not aligned for the vector kernels, have no shared grid: the
    bound step returns False and the caller issues the stages themselves."""
    world, n = 4, 64 * 4 * 50
    shard = n // world
    grad = gradient_like(n, torch.float32, 1, hip_device)
    send = torch.zeros(world, ops.payload_nbytes(shard), dtype=torch.uint8, device=hip_device)
    pairs = [ops.quant_pack(gradient_like(shard, torch.float32, 2 + r, hip_device)) for r in range(world)]
    mine = torch.zeros(ops.payload_nbytes(shard), dtype=torch.uint8, device=hip_device)
    quant = ops.bind_quant_pack_chunks(grad, send, world)
    reduce = ops.bind_dequant_reduce_quant(pairs, *ops.split_payload(mine, shard), shard)
    assert ops.bind_bucket_pipeline_step(quant, reduce)() is True
    # group 32
    send32 = torch.zeros(world, ops.payload_nbytes(shard, 32), dtype=torch.uint8, device=hip_device)
    pairs32 = [ops.quant_pack(gradient_like(shard, torch.float32, 2 + r, hip_device), group_size=32) for r in range(world)]
    mine32 = torch.zeros(ops.payload_nbytes(shard, 32), dtype=torch.uint8, device=hip_device)
    quant32 = ops.bind_quant_pack_chunks(grad, send32, world, group_size=32)
    reduce32 = ops.bind_dequant_reduce_quant(pairs32, *ops.split_payload(mine32, shard, 32), shard, group_size=32)
    assert ops.bind_bucket_pipeline_step(quant32, reduce32)() is False
    # a bucket that does not start on a 16-byte boundary
    shifted = torch.zeros(n + 1, device=hip_device)[1:]
    assert ops.bind_bucket_pipeline_step(ops.bind_quant_pack_chunks(shifted, send, world), reduce)() is False
    assert ops.bind_bucket_pipeline_step(quant, None, None)() is True       # one stage: its own kernel
    with pytest.raises(RuntimeError, match="at least one stage"):
        ops.bind_bucket_pipeline_step()
    with pytest.raises(RuntimeError, match="must come from bind_dequant_reduce_quant"):
        ops.bind_bucket_pipeline_step(quant, quant)


def test_pipeline_step_refuses_stages_that_write_into_each_other(ops, hip_device):
    """Nothing orders the stages inside the launch, so a stage that writes what another reads or writes is an error."""
    world, n = 8, 64 * 8 * 40
    shard = n // world
    nbytes = ops.payload_nbytes(shard)
    grad = gradient_like(n, torch.float32, 11, hip_device)
    send = torch.zeros(world, nbytes, dtype=torch.uint8, device=hip_device)
    gathered = torch.zeros(world, nbytes, dtype=torch.uint8, device=hip_device)
    mine = torch.zeros(nbytes, dtype=torch.uint8, device=hip_device)
    pairs = [ops.split_payload(send[r], shard) for r in range(world)]           # the reduce reads what the quantize writes
    quant = ops.bind_quant_pack_chunks(grad, send, world)
    reduce = ops.bind_dequant_reduce_quant(pairs, *ops.split_payload(mine, shard), shard)
    with pytest.raises(RuntimeError, match="another stage of the same launch"):
        ops.bind_bucket_pipeline_step(quant, reduce)()
    decode_into_the_input = ops.bind_dequant_chunks(gathered, grad, shard)      # the decode writes what the quantize reads
    with pytest.raises(RuntimeError, match="another stage of the same launch"):
        ops.bind_bucket_pipeline_step(quant, None, decode_into_the_input)()
    elsewhere = torch.zeros(n, device=hip_device)
    assert ops.bind_bucket_pipeline_step(quant, None, ops.bind_dequant_chunks(gathered, elsewhere, shard))() is True


def test_bucket_steps_dealt_to_two_streams_in_turn_equal_the_one_stream_schedule(ops, hip_device):
    """Consecutive buckets are independent: their launches (quantize of bucket k + reduce of bucket k-1) may alternate
    between two streams, each with its own send matrix and shard output, and must leave the same residuals, payloads
    and shards as the same launches on one stream."""
    world, n, buckets = 8, 64 * 8 * 500, 9
    shard = n // world
    stride = (ops.payload_nbytes(shard) + 255) // 256 * 256
    grads = [gradient_like(n, torch.bfloat16, 4000 + k, hip_device) for k in range(buckets)]
    start = [gradient_like(n, torch.float32, 4100 + k, hip_device, sigma=1e-5, outliers=False) for k in range(buckets)]
    peers = [[ops.quant_pack(gradient_like(shard, torch.float32, 4200 + 8 * k + r, hip_device)) for r in range(world)]
             for k in range(buckets)]

    def schedule(residuals, rows, outs):
        launches, previous = [], None
        for k in range(buckets):
            quant = ops.bind_quant_pack_chunks(grads[k], rows[k], world, residual=residuals[k], new_residual=residuals[k])
            reduce = ops.bind_dequant_reduce(peers[k], outs[k], divisor=float(world))
            launches.append(quant if previous is None else ops.bind_quant_chunks_and_reduce(quant, previous))
            previous = reduce
        return launches, previous

    def fresh():
        return ([r.clone() for r in start],
                [torch.zeros(world, stride, dtype=torch.uint8, device=hip_device) for _ in range(buckets)],
                [torch.empty(shard, device=hip_device) for _ in range(buckets)])

    want_residuals, want_rows, want_outs = fresh()
    launches, last = schedule(want_residuals, want_rows, want_outs)
    for launch in launches:
        assert launch() is True
    assert last() is True
    torch.cuda.synchronize()

    got_residuals, got_rows, got_outs = fresh()
    launches, last = schedule(got_residuals, got_rows, got_outs)
    from lowbit_comm_amd.hip import StreamLanes

    lanes = StreamLanes(2)
    assert len(lanes) == 2 and lanes.handle(0) != lanes.handle(1) and lanes.handle(2) == lanes.handle(0)
    assert lanes.stream(3).cuda_stream == lanes.handle(1)
    lanes.fork()
    for k, launch in enumerate(launches):
        assert launch(lanes.handle(k)) is True
    assert last(lanes.handle(buckets)) is True
    lanes.join()
    torch.cuda.synchronize()
    for k in range(buckets):
        assert torch.equal(got_rows[k], want_rows[k]), f"payloads of bucket {k}"
        assert_same_bits(got_residuals[k], want_residuals[k].cpu(), f"residual of bucket {k}")
        assert_same_bits(got_outs[k], want_outs[k].cpu(), f"shard of bucket {k}")


def test_shared_launch_reports_what_it_has_no_grid_for(ops, hip_device):
    n, world = 64 * 8 * 64, 8
    shard = n // world
    rows = torch.zeros(world, (ops.payload_nbytes(shard) + 255) // 256 * 256, dtype=torch.uint8, device=hip_device)
    peers8 = [ops.quant_pack(gradient_like(4096, torch.float32, 3300 + r, hip_device)) for r in range(8)]
    out = torch.empty(4096, device=hip_device)
    reduce8 = ops.bind_dequant_reduce(peers8, out)
    reduce3 = ops.bind_dequant_reduce(peers8[:3], out)
    bf16 = gradient_like(n, torch.bfloat16, 3301, hip_device)
    fp32 = gradient_like(n, torch.float32, 3302, hip_device)
    # a 16-bit residual, another group size: valid requests, no shared grid; any payload count up to eight has one
    half_residual = gradient_like(n, torch.bfloat16, 3304, hip_device, sigma=1e-5, outliers=False)
    assert ops.bind_quant_chunks_and_reduce(
        ops.bind_quant_pack_chunks(bf16, rows, world, residual=half_residual), reduce8)() is False
    assert ops.bind_quant_chunks_and_reduce(ops.bind_quant_pack_chunks(fp32, rows, world), reduce3)() is True
    rows32 = torch.zeros(world, (ops.payload_nbytes(shard, 32) + 255) // 256 * 256, dtype=torch.uint8, device=hip_device)
    peers32 = [ops.quant_pack(gradient_like(4096, torch.float32, 3310 + r, hip_device), group_size=32) for r in range(8)]
    assert ops.bind_quant_chunks_and_reduce(ops.bind_quant_pack_chunks(fp32, rows32, world, group_size=32),
                                            ops.bind_dequant_reduce(peers32, out, group_size=32))() is False
    # an unaligned view: element-wise kernels only
    odd = gradient_like(n + 1, torch.float32, 3303, hip_device)[1:]
    assert ops.bind_quant_chunks_and_reduce(ops.bind_quant_pack_chunks(odd, rows, world), reduce8)() is False
    # one side empty: the other runs alone
    empty = torch.empty(0, dtype=torch.float32, device=hip_device)
    no_rows = torch.zeros(world, 0, dtype=torch.uint8, device=hip_device)
    out.zero_()
    assert ops.bind_quant_chunks_and_reduce(ops.bind_quant_pack_chunks(empty, no_rows, world), reduce8)() is True
    want = torch.empty_like(out)
    assert ops.dequant_reduce_into(peers8, want)
    assert torch.equal(out.view(torch.int32), want.view(torch.int32))
    with pytest.raises(RuntimeError, match="bind_quant_pack_chunks"):
        ops.bind_quant_chunks_and_reduce(reduce8, reduce8)
    restored = torch.empty(n, device=hip_device)
    with pytest.raises(RuntimeError, match="restored"):
        ops.bind_quant_chunks_and_reduce(ops.bind_quant_pack_chunks(fp32, rows, world, restored=restored), reduce8)


# --------------------------------------------------------------------------- #
# seeded random sweep: sizes, start offsets, dtypes, rank counts and access modes nobody picked by hand
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_and_offsets_against_the_oracle(hip_device, seed):
    """Every case: a bucket view at a random element offset (so every alignment class of the kernels is met), split
    into a random number of chunks with or without a residual, quantized; then the same number of payloads reduced into
    a shard view - both against the oracle, bit for bit."""
    from lowbit_comm_amd.hip import ops as hip_ops

    rng = np.random.default_rng(4000 + seed)
    for case in range(40):
        dtype = str(rng.choice(["fp32", "bf16", "fp16"]))
        kind = DTYPES[dtype]
        world = int(rng.integers(1, 9))
        n = int(rng.choice([rng.integers(1, 200), rng.integers(200, 70_000), 64 * world * int(rng.integers(1, 400))]))
        offset = int(rng.integers(0, 9))
        group = int(rng.choice([64, 64, 64, 32, 16]))
        mode = str(rng.choice(["cached", "stream", "auto"]))
        with_residual = bool(rng.integers(0, 2))
        what = f"seed {seed} case {case}: {dtype} n={n} offset={offset} world={world} group={group} {mode} residual={with_residual}"
        grad = gradient_like(n + offset, kind, 9000 + 100 * seed + case, hip_device)[offset:]
        residual = None
        if with_residual:
            residual = gradient_like(n + offset, torch.float32, 9500 + case, hip_device, sigma=1e-5, outliers=False)[offset:]
        keep = None if residual is None else residual.clone()
        shard = -(-n // world)
        nbytes = hip_ops.payload_nbytes(shard, group)
        stride = (nbytes + 3) // 4 * 4 + 4 * int(rng.integers(0, 3))
        rows = torch.zeros(world, stride, dtype=torch.uint8, device=hip_device)
        with hip_ops.access_mode(mode):
            assert hip_ops.quant_pack_chunks_into(grad, rows, world, group_size=group, residual=residual,
                                                  new_residual=residual), what
        prepared = grad.cpu() if keep is None else grad.cpu() + keep.cpu()
        dropped = []
        for d in range(world):
            chunk = prepared[d * shard:(d + 1) * shard]
            if chunk.numel() < shard:
                chunk = torch.cat([chunk, torch.zeros(shard - chunk.numel(), dtype=chunk.dtype)])
            codes, scales = codec_torch.quantize(chunk, group)
            assert torch.equal(rows[d, :nbytes].cpu(), codec_torch.pack(codes, scales)), f"{what}: chunk {d}"
            dropped.append(chunk.float() - codec_torch.dequantize(codes, scales, shard, group, "fp32"))
        if residual is not None:
            assert_same_bits(residual, torch.cat(dropped)[:n], f"{what}: residual")
        # the chunk payloads, taken as what `world` peers sent for one shard, reduced into a view at another offset
        out_offset = int(rng.integers(0, 5))
        out = torch.zeros(shard + out_offset, dtype=kind, device=hip_device)[out_offset:]
        pairs = [hip_ops.split_payload(rows[d, :nbytes], shard, group) for d in range(world)]
        op = str(rng.choice(["sum", "mean"]))
        with hip_ops.access_mode(mode):
            assert hip_ops.dequant_reduce_into(pairs, out, group_size=group, divisor=float(world) if op == "mean" else 1.0), what
        want = codec_torch.reduce_payloads([(c.cpu(), s.cpu()) for c, s in pairs], shard, group, dtype, op)
        assert_same_bits(out, want, f"{what}: reduced shard ({op})")
