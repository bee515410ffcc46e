"""Pins for the CPU oracle: three independent restatements, exact-rational brute force,
invariants and the literal vectors held by the reference's own tests.

The reference has no golden INT8 codes/scales; what it holds for this path are literal
vectors for the packer (tests/test_payload_packing.py:12-57) and the error-feedback cycle
(tests/test_error_feedback.py:60-95).  Everything else is pinned by what IEEE-754 fixes.
"""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import codec_np, codec_torch, scalar

EPS_BITS = 0x34000000


# --------------------------------------------------------------------------- #
# exact-rational helpers (independent of numpy's float32 ops)
# --------------------------------------------------------------------------- #
def _round_to_f32(value: Fraction) -> np.float32:
    """Correctly rounded (nearest-even) float32 of an exact rational."""
    if value == 0:
        return np.float32(0.0)
    guess = np.float32(float(value))
    best = None
    for cand in (np.nextafter(guess, np.float32(-np.inf)), guess, np.nextafter(guess, np.float32(np.inf))):
        err = abs(Fraction(float(cand)) - value)
        even = (int(np.float32(cand).view(np.uint32)) & 1) == 0
        key = (err, 0 if even else 1)
        if best is None or key < best[0]:
            best = (key, np.float32(cand))
    return best[1]


def _rint_half_even(value: Fraction) -> int:
    floor = value.numerator // value.denominator
    frac = value - floor
    if frac > Fraction(1, 2):
        return floor + 1
    if frac < Fraction(1, 2):
        return floor
    return floor if floor % 2 == 0 else floor + 1


def _brute_quantize(values, group_size):
    values = [Fraction(float(np.float32(v))) for v in values]
    n = len(values)
    groups = -(-n // group_size)
    values = values + [Fraction(0)] * (groups * group_size - n)
    codes, scales = [], []
    for g in range(groups):
        chunk = values[g * group_size:(g + 1) * group_size]
        absmax = max(abs(v) for v in chunk)
        scale = _round_to_f32(absmax / 127)
        if scale < np.float32(2.0 ** -23):
            scale = np.float32(2.0 ** -23)
        scales.append(scale)
        for v in chunk:
            q = _round_to_f32(v / Fraction(float(scale)))
            codes.append(max(-127, min(127, _rint_half_even(Fraction(float(q))))))
    return np.array(codes, dtype=np.int8), np.array(scales, dtype=np.float32)


def _gradient_like(rng, n, sigma=1e-3, outliers=True):
    x = rng.standard_normal(n).astype(np.float32) * np.float32(sigma)
    if outliers and n:
        mask = rng.random(n) < 1e-3
        x[mask] = rng.standard_normal(int(mask.sum())).astype(np.float32) * np.float32(1e-1)
    return x


# --------------------------------------------------------------------------- #
# quantize
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("n,g", [(1, 64), (63, 64), (64, 64), (65, 64), (200, 64), (48, 16), (100, 32)])
def test_quantize_matches_exact_rational_brute_force(n, g):
    rng = np.random.default_rng(100 + n)
    x = _gradient_like(rng, n)
    codes, scales = codec_np.quantize(x, g)
    want_codes, want_scales = _brute_quantize(list(x), g)
    assert np.array_equal(scales.view(np.uint32), want_scales.view(np.uint32))
    assert np.array_equal(codes, want_codes)


@pytest.mark.parametrize("n", [0, 1, 64, 131, 4096, 100_003])
@pytest.mark.parametrize("g", [16, 32, 64])
def test_three_restatements_agree_on_fp32(n, g):
    rng = np.random.default_rng(7 * n + g)
    x = _gradient_like(rng, n)
    c_np, s_np = codec_np.quantize(x, g)
    c_c, s_c = scalar.quantize(x, g)
    c_t, s_t = codec_torch.quantize(torch.from_numpy(x), g)
    assert np.array_equal(c_np, c_c) and np.array_equal(c_np, c_t.numpy())
    assert np.array_equal(s_np.view(np.uint32), s_c.view(np.uint32))
    assert np.array_equal(s_np.view(np.uint32), s_t.numpy().view(np.uint32))
    assert c_np.size == -(-n // g) * g and s_np.size == -(-n // g)
    d_np = codec_np.dequantize(c_np, s_np, n, g)
    d_c = scalar.dequantize(c_c, s_c, n, g)
    d_t = codec_torch.dequantize(c_t, s_t, n, g).numpy()
    assert np.array_equal(d_np.view(np.uint32), d_c.view(np.uint32))
    assert np.array_equal(d_np.view(np.uint32), d_t.view(np.uint32))


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_numpy_and_torch_agree_on_16bit_inputs_and_outputs(dtype):
    gen = torch.Generator().manual_seed(5)
    t = (torch.randn(10_007, generator=gen) * 1e-3).to(codec_torch.torch_dtype(dtype))
    raw = t.view(torch.int16).numpy().view(np.uint16) if dtype == "bf16" else t.numpy()
    c_np, s_np = codec_np.quantize(codec_np.widen(raw, dtype), 64)
    c_t, s_t = codec_torch.quantize(t, 64)
    assert np.array_equal(c_np, c_t.numpy())
    assert np.array_equal(s_np.view(np.uint32), s_t.numpy().view(np.uint32))
    d_np = codec_np.dequantize(c_np, s_np, t.numel(), 64, dtype)
    d_t = codec_torch.dequantize(c_t, s_t, t.numel(), 64, dtype)
    d_t_raw = d_t.view(torch.int16).numpy().view(np.uint16) if dtype == "bf16" else d_t.numpy().view(np.uint16)
    assert np.array_equal(np.asarray(d_np).view(np.uint16), d_t_raw)


def test_bf16_rounding_matches_torch_including_ties_and_specials():
    rng = np.random.default_rng(3)
    x = rng.standard_normal(50_000).astype(np.float32)
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, 1.00390625, 1.01171875,
                        3.3895314e38, 1e-40, -1e-45], dtype=np.float32)
    ties = (np.arange(256, dtype=np.uint32) << 16 | 0x8000 | 0x3F800000).view(np.float32)
    x = np.concatenate([x, special, ties])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = codec_np.f32_to_bf16(x)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(codec_np.bf16_to_f32(got[nan])))
    assert np.array_equal(codec_np.bf16_to_f32(want[~nan]),
                          torch.from_numpy(want.view(np.int16)).view(torch.bfloat16).float().numpy()[~nan])


def test_round_half_to_even_on_exact_ties():
    # absmax 127 -> scale exactly 1.0, so the quotient is the value itself.
    x = np.zeros(64, dtype=np.float32)
    x[:9] = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, 126.5]
    codes, scales = codec_np.quantize(x, 64)
    assert scales[0] == np.float32(1.0)
    assert codes[:9].tolist() == [127, 0, 2, 2, 0, -2, -2, 4, 126]
    assert scalar.quantize(x, 64)[0][:9].tolist() == [127, 0, 2, 2, 0, -2, -2, 4, 126]


def test_true_division_not_reciprocal_multiply():
    """A quotient whose correctly rounded value is an exact tie while x*(1/s) is not."""
    rng = np.random.default_rng(11)
    found = 0
    for _ in range(4000):
        x = _gradient_like(rng, 64, outliers=False)
        scale = np.maximum(np.max(np.abs(x)) / np.float32(127.0), np.float32(2.0 ** -23))
        by_div = np.rint(x / scale)
        by_mul = np.rint(x * (np.float32(1.0) / scale))
        differs = by_div != by_mul
        if differs.any():
            found += 1
            codes, _ = codec_np.quantize(x, 64)
            brute, _ = _brute_quantize(list(x), 64)
            assert np.array_equal(codes, brute)
            assert np.array_equal(codes[differs], by_div[differs].astype(np.int8))
            if found >= 3:
                break
    assert found >= 1, "no reciprocal/division disagreement found: the pin is vacuous"


def test_zero_group_uses_eps_scale_and_zero_codes():
    x = np.zeros(128, dtype=np.float32)
    x[64] = 1e-3
    for quant in (codec_np.quantize, scalar.quantize):
        codes, scales = quant(x, 64)
        assert int(scales.view(np.uint32)[0]) == EPS_BITS
        assert not codes[:64].any()
        assert codes[64] == 127


def test_eps_clamp_applies_to_scale_not_absmax():
    x = np.zeros(64, dtype=np.float32)
    x[0], x[1], x[2] = 6e-7, -3.1e-7, 1.0e-7  # absmax/127 < eps
    codes, scales = codec_np.quantize(x, 64)
    assert int(scales.view(np.uint32)[0]) == EPS_BITS
    assert codes[:3].tolist() == [5, -3, 1]  # rint(x / 2^-23): 5.03, -2.60, 0.84
    assert np.array_equal(codes, scalar.quantize(x, 64)[0])


def test_denormal_inputs_are_not_flushed_before_the_division():
    x = np.full(64, 1e-40, dtype=np.float32)
    x[0] = 8e-8
    codes, scales = codec_np.quantize(x, 64)
    assert int(scales.view(np.uint32)[0]) == EPS_BITS
    assert codes[0] == 1 and not codes[1:].any()


@pytest.mark.parametrize("g", [16, 32, 64])
def test_quantize_invariants(g):
    rng = np.random.default_rng(17 + g)
    n = 50 * g + 7
    x = _gradient_like(rng, n)
    codes, scales = codec_np.quantize(x, g)
    groups = codes.reshape(-1, g).astype(np.int32)
    padded = np.zeros(groups.size, dtype=np.float32)
    padded[:n] = x
    rows = padded.reshape(-1, g)
    # the absmax element encodes to exactly +-127 with its own sign
    where = np.argmax(np.abs(rows), axis=1)
    peak = rows[np.arange(rows.shape[0]), where]
    assert np.array_equal(groups[np.arange(rows.shape[0]), where], np.sign(peak).astype(np.int32) * 127)
    assert np.abs(groups).max() == 127
    # padding encodes to zero
    assert not codes[n:].any()
    # half-step error bound (computed in float64, the bound has 2^-24 relative slack)
    err = np.abs(rows.astype(np.float64) - groups * scales.astype(np.float64)[:, None])
    assert np.all(err <= scales.astype(np.float64)[:, None] * (0.5 + 1e-6))
    # codes have the sign of the value
    assert np.all(groups * np.sign(rows) >= 0)


@pytest.mark.parametrize("k", [-5, -3, 1, 9, 40])
def test_power_of_two_equivariance(k):
    rng = np.random.default_rng(23)
    x = _gradient_like(rng, 64 * 40)
    codes, scales = codec_np.quantize(x, 64)
    scaled_codes, scaled_scales = codec_np.quantize(x * np.float32(2.0 ** k), 64)
    assert np.array_equal(codes, scaled_codes)
    assert np.array_equal(scaled_scales, scales * np.float32(2.0 ** k))


def test_requantizing_a_decoded_payload_is_idempotent():
    rng = np.random.default_rng(29)
    x = _gradient_like(rng, 64 * 100)
    codes, scales = codec_np.quantize(x, 64)
    decoded = codec_np.dequantize(codes, scales, x.size, 64)
    codes2, scales2 = codec_np.quantize(decoded, 64)
    assert np.array_equal(codes, codes2)
    assert np.allclose(scales, scales2, rtol=2e-7, atol=0)


def test_non_finite_policy():
    x = np.zeros(192, dtype=np.float32)
    x[0], x[1] = np.nan, 1.0
    x[64], x[65] = np.inf, 2.0
    x[128] = 1.0
    for quant in (codec_np.quantize, scalar.quantize, lambda a, g: tuple(
            t.numpy() for t in codec_torch.quantize(torch.from_numpy(a), g))):
        codes, scales = quant(x, 64)
        assert np.isnan(scales[0]) and np.isinf(scales[1]) and scales[2] == np.float32(1.0) / np.float32(127.0)
        assert not codes[:128].any()
        assert codes[128] == 127


# --------------------------------------------------------------------------- #
# dequantize + reduce
# --------------------------------------------------------------------------- #
def _payloads(rng, world, n, g=64):
    return [codec_np.quantize(_gradient_like(rng, n), g) for _ in range(world)]


@pytest.mark.parametrize("world", [1, 2, 3, 8])
def test_reduce_is_a_left_fold_in_list_order(world):
    rng = np.random.default_rng(41 + world)
    n = 64 * 6 + 5
    payloads = _payloads(rng, world, n)
    got = codec_np.reduce_payloads(payloads, n, 64, "fp32", "sum")
    want = np.empty(n, dtype=np.float32)
    for i in range(n):
        acc = None
        for codes, scales in payloads:
            term = _round_to_f32(Fraction(int(codes[i])) * Fraction(float(scales[i // 64])))
            acc = term if acc is None else _round_to_f32(Fraction(float(acc)) + Fraction(float(term)))
        want[i] = acc
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got.view(np.uint32), scalar.reduce_payloads(payloads, n, 64).view(np.uint32))
    t_payloads = [(torch.from_numpy(c), torch.from_numpy(s)) for c, s in payloads]
    assert np.array_equal(got.view(np.uint32),
                          codec_torch.reduce_payloads(t_payloads, n, 64).numpy().view(np.uint32))


def test_reduce_order_is_observable():
    rng = np.random.default_rng(43)
    n = 64 * 200
    payloads = _payloads(rng, 8, n)
    forward = codec_np.reduce_payloads(payloads, n)
    backward = codec_np.reduce_payloads(payloads[::-1], n)
    assert not np.array_equal(forward.view(np.uint32), backward.view(np.uint32))
    assert np.allclose(forward, backward, rtol=1e-5, atol=1e-9)


def test_mean_is_a_true_division_by_world_size():
    rng = np.random.default_rng(47)
    n = 64 * 50
    payloads = _payloads(rng, 3, n)
    total = codec_np.reduce_payloads(payloads, n, reduce="sum")
    mean = codec_np.reduce_payloads(payloads, n, reduce="mean")
    assert np.array_equal(mean, total / np.float32(3.0))
    assert not np.array_equal(mean, total * (np.float32(1.0) / np.float32(3.0)))
    assert np.array_equal(mean.view(np.uint32), scalar.reduce_payloads(payloads, n, 64, 3.0).view(np.uint32))
    t_payloads = [(torch.from_numpy(c), torch.from_numpy(s)) for c, s in payloads]
    assert np.array_equal(mean, codec_torch.reduce_payloads(t_payloads, n, 64, "fp32", "mean").numpy())


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_16bit_reduce_rounds_every_partial_sum(dtype):
    rng = np.random.default_rng(53)
    n = 64 * 30 + 3
    payloads = _payloads(rng, 4, n)
    t_payloads = [(torch.from_numpy(c), torch.from_numpy(s)) for c, s in payloads]
    for mode in ("sum", "mean"):
        got = codec_np.widen(codec_np.reduce_payloads(payloads, n, 64, dtype, mode), dtype)
        want = codec_torch.reduce_payloads(t_payloads, n, 64, dtype, mode).float().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_empty_payload_list_and_bad_mode_are_rejected():
    for mod in (codec_np, codec_torch):
        with pytest.raises(ValueError, match="empty payload list"):
            mod.reduce_payloads([], 0)
    with pytest.raises(ValueError, match="unsupported gather-reduce mode"):
        codec_np.reduce_payloads([codec_np.quantize(np.ones(64, np.float32))], 64, reduce="max")


# --------------------------------------------------------------------------- #
# wire format: a byte vector worked by hand from the two's-complement and IEEE-754 little-endian definitions (the
# reference's packer test checks a round trip and holds no bytes; that case is in tests/test_host_api.py)
# --------------------------------------------------------------------------- #
def test_pack_layout_literal_bytes(golden_vectors):
    vector = golden_vectors["packer_bytes_hand_computed"]
    assert vector["source"].startswith("NOT from the reference")
    codes = np.array(vector["codes"], dtype=np.int8)
    scales = np.array(vector["scales"], dtype=np.float32)
    packed = codec_np.pack(codes, scales)
    assert packed.dtype == np.uint8
    assert packed.tolist() == vector["packed_bytes"]
    assert codec_torch.pack(torch.from_numpy(codes), torch.from_numpy(scales)).tolist() == packed.tolist()


def test_pack_unpack_round_trip_and_size():
    rng = np.random.default_rng(59)
    x = _gradient_like(rng, 64 * 10 + 1)
    codes, scales = codec_np.quantize(x, 64)
    packed = codec_np.pack(codes, scales)
    assert packed.size == 11 * 68
    c2, s2 = codec_np.unpack(packed, 11, 64)
    assert np.array_equal(c2, codes) and np.array_equal(s2.view(np.uint32), scales.view(np.uint32))
    with pytest.raises(ValueError):
        codec_np.unpack(packed[:-1], 11, 64)


# --------------------------------------------------------------------------- #
# error feedback: literal vectors from the reference's tests
# --------------------------------------------------------------------------- #
def test_error_feedback_literal_cycle(golden_vectors):
    first = golden_vectors["error_feedback"]["update_then_compensate"]
    residual = codec_np.ef_residual(np.float32(first["original"]), np.float32(first["transmitted"]), "fp32")
    assert residual.tolist() == first["residual"]
    assert codec_np.ef_compensate(np.float32(first["next_gradient"]), "fp32", residual).tolist() == first["compensated"]
    cycle = golden_vectors["error_feedback"]["cycle"]
    r = codec_np.ef_residual(np.float32(cycle["original"]), np.float32(cycle["transmitted"]), "fp32")
    p = codec_np.ef_compensate(np.float32(cycle["gradient"]), "fp32", r)
    assert p.tolist() == cycle["compensated"]
    assert codec_np.ef_residual(p, np.float32(cycle["transmitted_next"]), "fp32").tolist() == cycle["residual_next"]


@pytest.mark.parametrize("restored_dtype", ["fp32", "bf16"])
def test_ef_round_trip_three_way(restored_dtype):
    gen = torch.Generator().manual_seed(61)
    n = 64 * 40 + 9
    grad = (torch.randn(n, generator=gen) * 1e-3).to(torch.bfloat16)
    residual = torch.randn(n, generator=gen) * 1e-5
    bits = grad.view(torch.int16).numpy().view(np.uint16)
    c_np, s_np, rest_np, res_np = codec_np.ef_round_trip(bits, "bf16", residual.numpy(), 64, restored_dtype)
    c_c, s_c, rest_c, res_c = scalar.ef_step_bf16(bits, residual.numpy(), 64, restored_dtype == "bf16")
    c_t, s_t, rest_t, res_t = codec_torch.ef_round_trip(grad, residual, 64, restored_dtype)
    assert res_t.dtype == torch.float32
    assert np.array_equal(c_np, c_c) and np.array_equal(c_np, c_t.numpy())
    assert np.array_equal(s_np.view(np.uint32), s_c.view(np.uint32))
    assert np.array_equal(s_np.view(np.uint32), s_t.numpy().view(np.uint32))
    assert np.array_equal(res_np.view(np.uint32), res_c.view(np.uint32))
    assert np.array_equal(res_np.view(np.uint32), res_t.numpy().view(np.uint32))
    rest_t_f = rest_t.float().numpy()
    assert np.array_equal(codec_np.widen(rest_np, restored_dtype), rest_t_f)
    assert np.array_equal(codec_np.widen(rest_c, restored_dtype), rest_t_f)
    # the residual is what quantization lost: |r'| <= scale/2 (+ bf16 rounding of restored)
    bound = np.repeat(s_np, 64)[:n].astype(np.float64) * 0.5
    if restored_dtype == "bf16":
        bound = bound + np.abs(rest_t_f).astype(np.float64) * 2.0 ** -8
    assert np.all(np.abs(res_np.astype(np.float64)) <= bound * (1 + 1e-6) + 1e-12)


def test_ef_residual_accumulates_over_steps():
    rng = np.random.default_rng(67)
    n = 64 * 20
    residual = None
    grads = []
    sent = np.zeros(n, dtype=np.float64)
    for _step in range(5):
        g = _gradient_like(rng, n)
        grads.append(g)
        codes, scales, restored, residual = codec_np.ef_round_trip(g, "fp32", residual)
        c2, s2, restored_c, residual_c = scalar.ef_step_f32(
            g, None if _step == 0 else prev_residual)  # noqa: F821
        assert np.array_equal(codes, c2) and np.array_equal(residual.view(np.uint32), residual_c.view(np.uint32))
        prev_residual = residual
        sent += restored.astype(np.float64)
    # telescoping: sum of transmitted + final residual == sum of gradients (up to fp32 rounding)
    assert np.allclose(sent + residual, np.sum(np.stack(grads).astype(np.float64), axis=0), rtol=0, atol=1e-8)


# --------------------------------------------------------------------------- #
# reduce-scatter / all-gather plan
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("n,world,want", [(10, 4, (3, 12)), (8, 8, (1, 8)), (0, 2, (0, 0)), (1, 8, (1, 8))])
def test_chunk_plan_shapes(n, world, want):
    shard, padded, ranges = codec_np.chunk_plan(n, world)
    assert (shard, padded) == want
    assert ranges == [(r * shard, (r + 1) * shard) for r in range(world)]


def test_chunk_plan_rejects_bad_arguments():
    with pytest.raises(ValueError):
        codec_np.chunk_plan(-1, 2)
    with pytest.raises(ValueError):
        codec_np.chunk_plan(4, 0)


def test_plan_restarts_groups_per_chunk_and_matches_a_direct_sum():
    rng = np.random.default_rng(71)
    world, n = 4, 64 * 9 + 30  # shard = 152 (not a multiple of 64): groups restart per chunk
    peers = [_gradient_like(rng, n) for _ in range(world)]
    shards, restored = codec_np.reduce_scatter_all_gather_plan(peers, 64, "sum")
    shard, _, ranges = codec_np.chunk_plan(n, world)
    assert all(s.size == shard for s in shards) and restored.size == n
    exact = np.sum(np.stack(peers).astype(np.float64), axis=0)
    padded = np.zeros(shard * world)
    padded[:n] = exact
    for d, (a, b) in enumerate(ranges):
        # W quantization errors of at most scale/2 each
        per_chunk_scale = max(np.max(np.abs(p[a:min(b, n)])) for p in peers) / 127 if a < n else 0
        assert np.all(np.abs(shards[d] - padded[a:b]) <= world * per_chunk_scale * 0.5 + 1e-9)
    # chunk d's first group starts at element a, not at a multiple of 64 of the bucket
    direct = codec_np.quantize(np.concatenate([peers[0], np.zeros(shard * world - n, np.float32)])[ranges[1][0]:ranges[1][1]], 64)
    assert np.array_equal(direct[0], codec_np.quantize_chunks(peers[0], world, 64)[1][0])
