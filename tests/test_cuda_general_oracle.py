"""Pins for the oracle of the reference's general CUDA kernels: code books, stochastic rounding, top-k side
channel, NaN-resetting maximum, rotated scan (oracle/cuda_wire_general_np.py, oracle/cuda_wire_general_scalar.c).

The reference never checks the output of these policies, so the restatements are pinned by what fixes them from
outside: the Philox known-answer vectors of the Random123 distribution, closed forms of the code books, exact
rational arithmetic, properties (nearest code, exact restoration of the top-k elements, unbiasedness), hand-worked
cases for the tie and NaN rules, literal bytes for the layout, and two independent implementations against each
other.  Agreement with an actual NVIDIA build stays unpinned.
"""
from __future__ import annotations

import itertools
from fractions import Fraction

import numpy as np
import pytest
from scipy.stats import norm

from oracle import cuda_wire_general_np as general
from oracle import cuda_wire_general_scalar as general_c
from oracle import cuda_wire_np as wire

DTYPES = ("fp32", "fp16", "bf16")
NUMPY = {"fp32": np.float32, "fp16": np.float16, "bf16": np.uint16}


def make(rng, n, dtype, sigma=1.0):
    return wire.from_f32((rng.standard_normal(n) * sigma).astype(np.float32), dtype)


def same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.tobytes() == b.tobytes()


# --------------------------------------------------------------------------- #
# Philox4x32-10 and the cuRAND stream
# --------------------------------------------------------------------------- #
def test_philox_known_answers(golden_vectors):
    """kat_vectors of the Random123 distribution, philox4x32 with 10 rounds (tests/golden/reference_vectors.json)."""
    vectors = golden_vectors["philox4x32_10"]["vectors"]
    assert len(vectors) == 3
    for vector in vectors:
        counter = tuple(int(word, 16) for word in vector["counter"])
        key = tuple(int(word, 16) for word in vector["key"])
        expected = tuple(int(word, 16) for word in vector["output"])
        got = general.philox4x32_10([np.array([c]) for c in counter], [np.array([k]) for k in key])
        assert tuple(int(word[0]) for word in got) == expected
        assert tuple(int(word) for word in general_c.philox_block(counter, key)) == expected


@pytest.mark.parametrize("offset", (0, 1, 2, 3, 4, 4099, 2 ** 34 + 6))
def test_stream_is_counter_mode(offset):
    """Draw j of subsequence s at offset o is word (o + j) % 4 of the block whose counter is ((o + j) / 4, s)."""
    seed, subsequences = 0x0123456789ABCDEF, [0, 5, 2 ** 32 + 9]
    draws = general.curand_draws(seed, np.array(subsequences), offset, 11)
    for row, s in enumerate(subsequences):
        assert (general_c.curand_draws(seed, s, offset, 11) == draws[row]).all()
        for j in range(11):
            block = (offset + j) // 4
            counter = (block & 0xFFFFFFFF, block >> 32, s & 0xFFFFFFFF, s >> 32)
            words = general_c.philox_block(counter, (seed & 0xFFFFFFFF, seed >> 32))
            assert int(draws[row, j]) == int(words[(offset + j) % 4])


def test_uniform_mapping():
    """(0, 1]: 0 -> 2^-33, 2^32 - 1 -> 1, the midpoint of the integer range -> 0.5 + 2^-33 rounded."""
    got = general.curand_uniform(np.array([0, 2 ** 32 - 1, 2 ** 31, 1], dtype=np.uint32))
    assert got.dtype == np.float32
    assert got[0] == np.float32(2.0 ** -33) and got[1] == np.float32(1.0) and got[2] == np.float32(0.5)
    assert got[3] == np.float32(1.5 * 2.0 ** -32)
    many = general.curand_uniform(general.curand_draws(99, np.arange(4096), 0, 64))
    assert many.min() > 0.0 and many.max() <= 1.0
    assert abs(float(many.mean()) - 0.5) < 3 * (1 / 12 / many.size) ** 0.5


# --------------------------------------------------------------------------- #
# code books
# --------------------------------------------------------------------------- #
def test_code_books_have_their_closed_forms():
    k = np.arange(-7, 8)
    assert np.abs(general.CODE_BOOKS["uniform"][:15] - k / 7.0).max() < 6e-8
    # equal steps in probability between the standard normal's -1 and +1 sigma points
    normal = norm.ppf(0.5 + k * (norm.cdf(1.0) - 0.5) / 7.0)
    assert np.abs(general.CODE_BOOKS["normal"][:15] - normal).max() < 6e-8
    powers = np.array([2.0 ** -e for e in range(7)], dtype=np.float32)
    assert (general.CODE_BOOKS["e3m0"][8:15] == powers[::-1]).all()
    e2m1 = np.array([1 / 8, 1 / 6, 1 / 4, 1 / 3, 1 / 2, 2 / 3, 1], dtype=np.float32)
    assert (general.CODE_BOOKS["e2m1"][8:15] == e2m1).all()
    for book in general.CODE_BOOKS.values():
        assert book[7] == 0 and np.isinf(book[15]) and (book[:7] == -book[8:15][::-1]).all()
        assert (np.diff(book[:15]) > 0).all()


@pytest.mark.parametrize("quant_type", tuple(general.CODE_BOOKS))
@pytest.mark.parametrize("dtype", DTYPES)
def test_code_book_codes_are_the_nearest_entries(quant_type, dtype):
    """Against exact rational arithmetic: the code is the entry nearest to t = fl(v / scale); inputs whose t lies
    within 1e-6 of a midpoint are left out (there the float32 subtraction decides)."""
    rng = np.random.default_rng(11)
    g = 16
    x = make(rng, g * 40, dtype)
    payload = general.quantize(x, dtype, g, 4, quant_type)
    codes, meta = general.split(payload, x.size, dtype, g, 4, 0, False)
    values = wire.to_f32(x, dtype).reshape(-1, g)
    book = [Fraction(float(entry)) for entry in general.CODE_BOOKS[quant_type][:15]]
    checked = 0
    for row in range(values.shape[0]):
        scale = np.float32(np.abs(values[row]).max())
        assert general._bits_to_f32(meta[row, :1], dtype)[0] == scale
        for i in range(g):
            t = Fraction(float(np.float32(values[row, i]) / np.float32(max(scale, np.float32(1e-6)))))
            distance = [abs(t - entry) for entry in book]
            best = min(range(15), key=lambda c: (distance[c], c))
            runner_up = sorted(distance)[1]
            if runner_up - distance[best] < Fraction(1, 10 ** 6):
                continue
            assert int(codes[row, i]) & 15 == best
            checked += 1
    assert checked > g * 35
    decoded = wire.to_f32(general.dequantize(payload, x.size, dtype, g, 4, quant_type), dtype).reshape(-1, g)
    expect = general.CODE_BOOKS[quant_type][codes.astype(np.int64) & 15] * np.abs(values).max(axis=1, keepdims=True)
    assert same_bits(wire.from_f32(expect.astype(np.float32).reshape(-1), dtype),
                     wire.from_f32(decoded.reshape(-1), dtype))


def test_midpoints_stay_on_the_lower_entry():
    """e3m0's midpoints are exact in float32: 0.75 lies halfway between 0.5 and 1.0 and keeps 0.5."""
    x = np.zeros(16, dtype=np.float32)
    x[:6] = [1.0, 0.75, 0.7500001, 0.375, -0.75, -0.7500001]
    for module in (general, general_c):
        codes, _ = general.split(module.quantize(x, "fp32", 16, 4, "e3m0"), 16, "fp32", 16, 4, 0, False)
        assert [int(c) & 15 for c in codes[0, :6]] == [14, 13, 14, 12, 0, 0]


# --------------------------------------------------------------------------- #
# top-k side channel
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("topk", (1, 2))
@pytest.mark.parametrize("compact", (False, True))
def test_top_k_elements_travel_verbatim(dtype, topk, compact):
    rng = np.random.default_rng(5)
    g = 32
    x = make(rng, g * 50, dtype)
    values = wire.to_f32(x, dtype).reshape(-1, g)
    payload = general.quantize(x, dtype, g, 8, "linear", topk, None, compact)
    assert payload.size == general.payload_nbytes(x.size, g, dtype, 8, topk)
    codes, meta = general.split(payload, x.size, dtype, g, 8, topk, compact)
    decoded = wire.to_f32(general.dequantize(payload, x.size, dtype, g, 8, "linear", topk, compact), dtype).reshape(-1, g)
    for row in range(values.shape[0]):
        magnitude = np.abs(values[row])
        if np.unique(magnitude).size < g:        # ties are covered by the hand-worked cases below
            continue
        order = np.argsort(-magnitude)
        indices = [int(meta[row, 1]) & 0xFF] + ([int(meta[row, 1]) >> 8] if topk == 2 else [])
        assert indices == [int(i) for i in order[:topk]]
        scale = general._bits_to_f32(meta[row, :1], dtype)[0]
        assert scale == magnitude[order[topk]]                       # the next largest magnitude
        for i in indices:
            assert decoded[row, i] == values[row, i] and codes[row, i] == 0
        rest = np.setdiff1d(np.arange(g), indices)
        assert np.abs(codes[row, rest]).max() == 127
        bound = scale / 254 * 1.0001 + np.abs(decoded[row, rest]) * 2.0 ** (-8 if dtype == "bf16" else -11)
        assert (np.abs(decoded[row, rest] - values[row, rest]) <= bound).all()


def test_top_k_ties_and_degenerate_groups_fp32():
    """fp32 kernels compare with >=: among equal magnitudes the later element wins, zeros qualify."""
    g = 16
    x = np.zeros(3 * g, dtype=np.float32)
    x[[2, 9]] = [3.0, -3.0]                                   # group 0: a tie for the largest
    x[g + 4] = 1.5                                            # group 1: a single non-zero
    x[2 * g:] = np.nan                                        # group 2: nothing comparable
    x[2 * g + 1] = np.float32(np.nan)
    for module in (general, general_c):
        _, meta = general.split(module.quantize(x, "fp32", g, 8, "linear", 2), x.size, "fp32", g, 8, 2, False)
        assert [int(meta[0, 1]) & 0xFF, int(meta[0, 1]) >> 8] == [9, 2]
        assert meta[0, 2:].view(np.float32).tolist() == [-3.0, 3.0] and meta[0, 0] == 0   # third largest is 0
        # one non-zero: it is first, the last zero of the scan (>= holds for 0 >= 0) is second
        assert [int(meta[1, 1]) & 0xFF, int(meta[1, 1]) >> 8] == [4, 15]
        assert [int(meta[2, 1]) & 0xFF, int(meta[2, 1]) >> 8] == [0, 1] and meta[2, 0] == 0
        _, meta = general.split(module.quantize(x, "fp32", g, 8, "linear", 1), x.size, "fp32", g, 8, 1, False)
        assert int(meta[0, 1]) == 9 and meta[0, :1].view(np.float32)[0] == 3.0
        assert int(meta[1, 1]) == 4 and meta[1, 0] == 0
        assert int(meta[2, 1]) == 0 and np.isnan(meta[2, :1].view(np.float32)[0])    # scale := element 1 as stored


def test_top_k_ties_and_degenerate_groups_16bit():
    """16-bit kernels compare with > in the rotated scan: the first equal magnitude of the scan wins, zeros never
    qualify.  Group 8 of a g=16 payload starts its scan at element 4."""
    g = 16
    x = np.zeros(10 * g, dtype=np.float16)
    x[[2, 9]] = [3.0, -3.0]                                   # group 0 (scan from 0): element 2 comes first
    x[8 * g + 2], x[8 * g + 9] = 3.0, -3.0                    # group 8 (scan from 4): element 9 comes first
    x[9 * g + 4] = 1.5                                        # group 9: a single non-zero
    for module in (general, general_c):
        _, meta = general.split(module.quantize(x, "fp16", g, 8, "linear", 2), x.size, "fp16", g, 8, 2, False)
        assert [int(meta[0, 1]) & 0xFF, int(meta[0, 1]) >> 8] == [2, 9]
        assert [int(meta[8, 1]) & 0xFF, int(meta[8, 1]) >> 8] == [9, 2]
        assert [int(meta[9, 1]) & 0xFF, int(meta[9, 1]) >> 8] == [4, 5] and meta[9, 0] == 0
        assert [int(meta[1, 1]) & 0xFF, int(meta[1, 1]) >> 8] == [0, 1]              # all zero


def test_scan_start_rotation():
    assert general.scan_start(np.arange(40), 64, "fp32").tolist() == [0] * 40
    assert general.scan_start(np.array([0, 1, 2, 3, 31, 32, 33]), 64, "bf16").tolist() == [0, 0, 4, 4, 60, 0, 0]
    assert general.scan_start(np.array([0, 3, 4, 31]), 32, "fp16").tolist() == [0, 0, 4, 28]
    assert general.scan_start(np.array([0, 7, 8, 31]), 16, "fp16").tolist() == [0, 0, 4, 12]


# --------------------------------------------------------------------------- #
# the NaN-resetting maximum
# --------------------------------------------------------------------------- #
def test_a_nan_resets_the_running_maximum():
    g = 16
    x = np.full(3 * g, 0.25, dtype=np.float32)
    x[0], x[1], x[2] = 5.0, np.nan, 3.0                       # group 0: only what follows the NaN counts
    x[g + 15] = np.nan                                        # group 1: the NaN is last, the scale is NaN
    x[2 * g + 3] = 7.0                                        # group 2: no NaN
    for module in (general, general_c):
        payload = module.quantize(x, "fp32", g)
        codes, meta = general.split(payload, x.size, "fp32", g, 8, 0, False)
        scales = meta[:, 0].view(np.float32)
        assert scales[0] == 3.0 and np.isnan(scales[1]) and scales[2] == 7.0
        assert codes[0, :3].tolist() == [127, 0, 127] and not codes[1].any()
    # 16-bit tensors scan group 8 of a g=16 payload from element 4: a NaN at element 5 hides element 4 only
    x16 = np.full(9 * g, 0.25, dtype=np.float16)
    x16[8 * g + 4], x16[8 * g + 5], x16[8 * g + 0] = 9.0, np.nan, 2.0
    for module in (general, general_c):
        _, meta = general.split(module.quantize(x16, "fp16", g), x16.size, "fp16", g, 8, 0, False)
        assert meta[8, :1].view(np.float16)[0] == 2.0


# --------------------------------------------------------------------------- #
# stochastic rounding
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", ("fp32", "bf16"))
def test_stochastic_linear_rounds_to_a_neighbour_and_is_unbiased(dtype):
    rng = np.random.default_rng(2)
    g = 64
    x = make(rng, g * 8, dtype)
    values = wire.to_f32(x, dtype).reshape(-1, g)
    scale = np.abs(values).max(axis=1, keepdims=True)
    exact = values.astype(np.float64) * (127.0 / scale)
    total = np.zeros_like(exact)
    trials = 400
    for trial in range(trials):
        payload = general.quantize(x, dtype, g, 8, "linear", 0, (1000 + trial, 4 * trial))
        codes, _ = general.split(payload, x.size, dtype, g, 8, 0, False)
        assert ((codes >= np.floor(exact - 1e-3)) & (codes <= np.ceil(exact + 1e-3))).all()
        total += codes
    # the mean code estimates v * 127 / scale with variance <= 1/4 per trial
    assert np.abs(total / trials - exact).max() < 5 * 0.5 / trials ** 0.5
    assert abs(float((total / trials - exact).mean())) < 5 * 0.5 / (trials * exact.size) ** 0.5


def test_stochastic_code_book_picks_the_upper_entry_with_the_right_probability():
    g = 64
    x = np.full(g * 64, 0.3, dtype=np.float32)
    x[::g] = 1.0                                              # scale 1, t = 0.3 between 0.25 and 0.5 of e3m0
    ups = []
    for trial in range(40):
        codes, _ = general.split(general.quantize(x, "fp32", g, 4, "e3m0", 0, (trial, 0)), x.size, "fp32", g, 4, 0, False)
        picked = codes.reshape(-1, g)[:, 1:] & 15
        assert set(np.unique(picked)) <= {12, 13}
        ups.append((picked == 13).mean())
    expected = (0.3 - 0.25) / 0.25
    assert abs(float(np.mean(ups)) - expected) < 5 * (expected * (1 - expected) / (40 * 63 * 64)) ** 0.5


def test_the_same_seed_gives_the_same_payload_and_another_offset_does_not():
    x = make(np.random.default_rng(3), 64 * 20, "fp16")
    a = general.quantize(x, "fp16", 64, 8, "linear", 0, (17, 128))
    assert same_bits(a, general.quantize(x, "fp16", 64, 8, "linear", 0, (17, 128)))
    assert not same_bits(a, general.quantize(x, "fp16", 64, 8, "linear", 0, (17, 132)))
    assert not same_bits(a, general.quantize(x, "fp16", 64, 8, "linear", 0, (18, 128)))


# --------------------------------------------------------------------------- #
# layout and sizes
# --------------------------------------------------------------------------- #
def test_payload_sizes():
    """gen_code_quant.py:167-178: +8 / +12 bytes per group for fp32, +4 / +6 for 16-bit."""
    assert general.payload_nbytes(64, 64, "fp32", 8, 0) == 68 and general.payload_nbytes(64, 64, "fp32", 8, 1) == 76
    assert general.payload_nbytes(64, 64, "fp32", 8, 2) == 80 and general.payload_nbytes(64, 64, "bf16", 4, 1) == 38
    assert general.payload_nbytes(640, 64, "fp16", 8, 2) == 10 * 72 and general.payload_nbytes(0, 64, "fp16", 8, 2) == 0


def test_literal_bytes_with_two_outliers():
    """One fp32 group of 16 and one fp16 group of 16, k = 2, written out by hand."""
    x = np.zeros(16, dtype=np.float32)
    x[0], x[3], x[5], x[6] = 1.0, -8.0, 0.5, 16.0            # outliers 16 (index 6), -8 (index 3); scale 1.0
    want_codes = [0, 0, 0, 127, 0, 0, 64, 0] + [0] * 8       # words of 4 codes, first code in the top byte
    #             word0 = [127,0,0,0] reversed            word1 = [0,64,0,0] reversed (0.5*127 = 63.5 -> 64)
    meta = np.array([1.0], dtype=np.float32).tobytes() + (6 | (3 << 8)).to_bytes(4, "little") \
        + np.array([16.0, -8.0], dtype=np.float32).tobytes()
    for module in (general, general_c):
        payload = module.quantize(x, "fp32", 16, 8, "linear", 2, None, True)
        assert payload.tobytes() == bytes(want_codes) + meta
        assert same_bits(module.dequantize(payload, 16, "fp32", 16, 8, "linear", 2, True)[[0, 3, 5, 6]],
                         np.array([1.0, -8.0, np.float32(64) * (np.float32(1.0) / np.float32(127.0)), 16.0], dtype=np.float32))
    h = x.astype(np.float16)
    meta16 = np.array([1.0], dtype=np.float16).tobytes() + (6 | (3 << 8)).to_bytes(2, "little") \
        + np.array([16.0, -8.0], dtype=np.float16).tobytes()
    want16 = [0, 127, 0, 0, 64, 0, 0, 0] + [0] * 8           # words of 2 codes: [127,0] [0,0] [0,64] [0,0] reversed
    for module in (general, general_c):
        assert module.quantize(h, "fp16", 16, 8, "linear", 2, None, False).tobytes() == bytes(want16) + meta16


# --------------------------------------------------------------------------- #
# two implementations
# --------------------------------------------------------------------------- #
def _policies():
    for bit, topk, compact, stochastic in itertools.product((4, 8), (0, 1, 2), (False, True), (None, (42, 8), (7, 3))):
        for quant_type in (general.QUANT_TYPES if bit == 4 else ("linear",)):
            yield bit, quant_type, topk, compact, stochastic


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("g", (16, 32, 64))
def test_numpy_and_c_restatements_agree(dtype, g):
    rng = np.random.default_rng(g)
    for case, (bit, quant_type, topk, compact, stochastic) in enumerate(_policies()):
        values = (rng.standard_normal(g * 70) * rng.choice([1e-7, 1e-3, 1.0, 100.0])).astype(np.float32)
        values[rng.integers(0, values.size, 24)] = 0.0
        if case % 3 == 0:
            values[rng.integers(0, values.size, 6)] = np.nan
            values[rng.integers(0, values.size, 3)] = np.inf
            values[g:2 * g] = np.nan                                  # a group of NaNs
            values[2 * g:3 * g] = 0.0                                 # a group of zeros
            values[3 * g:4 * g] = -2.5                                # a group of equal values
        x = wire.from_f32(values, dtype)
        a = general.quantize(x, dtype, g, bit, quant_type, topk, stochastic, compact)
        b = general_c.quantize(x, dtype, g, bit, quant_type, topk, stochastic, compact)
        assert same_bits(a, b), (bit, quant_type, topk, compact, stochastic)
        out = make(rng, values.size, dtype)
        for op in ("none", "sum", "max", "min"):
            da = general.dequantize(a, values.size, dtype, g, bit, quant_type, topk, compact, op, out)
            db = general_c.dequantize(a, values.size, dtype, g, bit, quant_type, topk, compact, op, out)
            assert same_bits(da, db), (bit, quant_type, topk, compact, op)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bit", (4, 8))
@pytest.mark.parametrize("compact", (False, True))
def test_plain_linear_policy_matches_the_pack_kernel_restatement_on_finite_input(dtype, bit, compact):
    """Without NaNs the general kernels and the fused pack kernel write the same bytes."""
    x = make(np.random.default_rng(8), 64 * 33, dtype, 0.02)
    assert same_bits(general.quantize(x, dtype, 64, bit, "linear", 0, None, compact),
                     wire.quantize(x, dtype, 64, compact, None, bit))
    payload = wire.quantize(x, dtype, 64, compact, None, bit)
    assert same_bits(general.dequantize(payload, x.size, dtype, 64, bit, "linear", 0, compact),
                     wire.dequantize(payload, x.size, dtype, 64, compact, "none", None, bit))
