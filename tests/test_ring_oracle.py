"""Pins of the ring all-reduce oracle (oracle/ring_np.py): brute force, lossless inputs with a known exact answer,
the message-passing invariants of a ring and an error bound.  CPU only."""
import struct

import numpy as np
import pytest

from oracle import codec_np, ring_np


def f32(value: float) -> float:
    return struct.unpack("<f", struct.pack("<f", value))[0]


def brute_force_step(codes, scales, chunk, g, accumulate, divisor):
    """Python floats (binary64) rounded to binary32 after every operation: each of the operations here (product
    of a small integer and a float32, sum, quotient of two float32) is exactly representable or correctly rounded
    in binary64 before the final rounding, so this equals float32 arithmetic."""
    out = []
    for i, old in enumerate(chunk):
        value = f32(float(codes[i]) * float(scales[i // g]))
        if accumulate:
            value = f32(float(old) + value)
        if divisor != 1.0:
            value = f32(value / divisor)
        out.append(value)
    padded = out + [0.0] * (-len(out) % g)
    payload_codes, payload_scales = [], []
    for start in range(0, len(padded), g):
        group = padded[start:start + g]
        scale = max(f32(max(abs(v) for v in group) / 127.0), 2.0 ** -23)
        payload_scales.append(scale)
        for v in group:
            q = f32(v / scale)
            r = float(np.rint(q))
            payload_codes.append(int(max(-127.0, min(127.0, r))))
    return out, payload_codes, payload_scales


@pytest.mark.parametrize("accumulate, divisor", [(True, 1.0), (True, 3.0), (False, 1.0), (True, 8.0)])
def test_ring_step_matches_python_float_brute_force(accumulate, divisor):
    rng = np.random.default_rng(7)
    g, n = 16, 37
    incoming = rng.standard_normal(n).astype(np.float32)
    codes, scales = codec_np.quantize(incoming, g)
    chunk = (rng.standard_normal(n) * 0.5).astype(np.float32)
    new_chunk, payload = ring_np.ring_step((codes, scales), chunk, "fp32", g,
                                           reduce_op="sum" if accumulate else "none", divisor=divisor)
    want, want_codes, want_scales = brute_force_step(codes.tolist(), scales.tolist(), chunk.tolist(), g, accumulate,
                                                     divisor)
    assert new_chunk.tolist() == want
    assert payload[0].tolist() == want_codes
    assert payload[1].tolist() == want_scales


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
def test_ring_step_is_decode_then_add_then_divide_then_quantize(dtype):
    rng = np.random.default_rng(11)
    g, n = 32, 200
    codes, scales = codec_np.quantize(rng.standard_normal(n).astype(np.float32), g)
    chunk = codec_np.narrow(rng.standard_normal(n).astype(np.float32), dtype)
    new_chunk, payload = ring_np.ring_step((codes, scales), chunk, dtype, g, reduce_op="sum", divisor=5.0)
    decoded = codec_np.widen(codec_np.dequantize(codes, scales, n, g, dtype), dtype)
    summed = codec_np.widen(codec_np.narrow(codec_np.widen(chunk, dtype) + decoded, dtype), dtype)
    mean = codec_np.narrow(summed / np.float32(5.0), dtype)
    assert np.array_equal(new_chunk, mean)
    want_codes, want_scales = codec_np.quantize(codec_np.widen(mean, dtype), g)
    assert np.array_equal(payload[0], want_codes) and np.array_equal(payload[1], want_scales)
    # reduce op "none" ignores what the chunk held
    over, _ = ring_np.ring_step((codes, scales), chunk, dtype, g, reduce_op="none")
    assert np.array_equal(over, codec_np.dequantize(codes, scales, n, g, dtype))
    with pytest.raises(ValueError):
        ring_np.ring_step((codes, scales), chunk, dtype, g, reduce_op="max")


def lossless_buckets(world, n, g, rng):
    """Per chunk-local group every rank holds +-127 * 2^j * k_rank with the signs shared between ranks, so that
    every payload on the way has codes +-127 and a scale 2^j * K that decodes exactly."""
    _shard, _padded, ranges = codec_np.chunk_plan(n, world)
    signs = rng.choice(np.array([-1.0, 1.0], dtype=np.float32), size=n)
    exponents = np.zeros(n, dtype=np.int64)
    factors = np.ones((world, n), dtype=np.int64)
    for a, b in ranges:
        a, b = min(a, n), min(b, n)
        if b <= a:
            continue
        local = np.arange(b - a) // g
        groups = int(local[-1]) + 1
        exponents[a:b] = rng.integers(-12, 4, size=groups)[local]
        for rank in range(world):
            factors[rank, a:b] = rng.integers(1, 6, size=groups)[local]
    base = signs * np.float32(127.0) * np.exp2(exponents).astype(np.float32)
    buckets = [(base * factors[rank].astype(np.float32)).astype(np.float32) for rank in range(world)]
    exact_sum = base.astype(np.float64) * factors.sum(axis=0)
    return buckets, exact_sum


@pytest.mark.parametrize("world, n, g", [(2, 64 * 6, 64), (4, 64 * 8 + 40, 64), (8, 16 * 41 + 3, 16), (8, 8 * 64, 64),
                                          (4, 7, 16), (8, 5, 16)])
def test_ring_all_reduce_returns_the_exact_mean_when_every_quantization_is_lossless(world, n, g):
    rng = np.random.default_rng(world * 1000 + n)
    buckets, exact_sum = lossless_buckets(world, n, g, rng)
    results = ring_np.ring_all_reduce(buckets, "fp32", g)
    want = (exact_sum / world).astype(np.float32)
    assert np.array_equal(want.astype(np.float64), exact_sum / world)       # representable: the test is exact
    assert len(results) == world
    for rank in range(world):
        assert np.array_equal(results[rank], want), rank
    for rank in range(world):                                               # inputs are not touched
        assert buckets[rank] is not results[rank]


@pytest.mark.parametrize("world", [3, 5, 7])
def test_ring_all_reduce_divides_the_complete_sum_once_on_the_owner(world):
    """Not a power of two: the mean is rounded, so only the owner's unquantized chunk is exact; every other rank
    holds that chunk quantized once and decoded."""
    g, n = 16, world * 48
    rng = np.random.default_rng(world)
    buckets, exact_sum = lossless_buckets(world, n, g, rng)
    results = ring_np.ring_all_reduce(buckets, "fp32", g)
    shard = n // world
    mean = (exact_sum.astype(np.float32) / np.float32(world)).astype(np.float32)
    for owner in range(world):
        a, b = owner * shard, (owner + 1) * shard
        assert np.array_equal(results[owner][a:b], mean[a:b])
        codes, scales = codec_np.quantize(mean[a:b], g)
        travelled = codec_np.dequantize(codes, scales, shard, g, "fp32")
        again = travelled
        for hop in range(1, world):
            # the payload is re-quantized at every hop (pipelined_ring.py:250-254); follow it
            rank = (owner + hop) % world
            assert np.array_equal(results[rank][a:b], again), (owner, rank)
            codes, scales = codec_np.quantize(again, g)
            again = codec_np.dequantize(codes, scales, shard, g, "fp32")


def test_world_of_one_leaves_the_bucket_alone_and_empty_buckets_work():
    x = np.arange(10, dtype=np.float32)
    assert np.array_equal(ring_np.ring_all_reduce([x], "fp32", 16)[0], x)
    empty = ring_np.ring_all_reduce([np.zeros(0, np.float32)] * 3, "fp32", 16)
    assert all(r.size == 0 for r in empty)


@pytest.mark.parametrize("dtype", ["fp32", "bf16", "fp16"])
def test_ring_all_reduce_stays_within_the_bound_of_successive_quantizations(dtype):
    world, n, g = 8, 8 * 64 * 3 + 17, 64
    rng = np.random.default_rng(5)
    raw = [rng.standard_normal(n).astype(np.float32) * 1e-3 for _ in range(world)]
    buckets = [codec_np.narrow(b, dtype) for b in raw]
    exact = np.mean([codec_np.widen(b, dtype).astype(np.float64) for b in buckets], axis=0)
    results = ring_np.ring_all_reduce(buckets, dtype, g)
    peak = sum(float(np.max(np.abs(codec_np.widen(b, dtype)))) for b in buckets)    # bounds every partial sum
    # W-1 quantizations of partial sums (each off by at most scale/2 <= peak/254) divided by W, up to W-1 more
    # of the mean on the way round, plus the roundings of decodes and sums in the bucket's own type
    type_eps = {"fp32": 2.0 ** -24, "bf16": 2.0 ** -8, "fp16": 2.0 ** -11}[dtype]
    bound = 2 * (world - 1) * peak / 254 / world + 4 * world * type_eps * peak
    for rank in range(world):
        error = np.max(np.abs(codec_np.widen(results[rank], dtype).astype(np.float64) - exact))
        assert error <= bound, (rank, error, bound)
        assert error > 0


@pytest.mark.parametrize("world", [2, 3, 5, 8])
def test_messages_follow_the_ring_the_reference_tests_describe(world):
    """Expectations stated in the reference's own schedule tests (tests/cuda/test_topology_executors.py:622-714):
    every rank sends to rank+1 and receives from rank-1; at reduce step s it sends chunk (rank-s-1) mod W and
    receives chunk (rank-s-2) mod W, the last one being its own; at gather step s it sends chunk (rank-s) mod W
    and receives chunk (rank-s-1) mod W; every rank ends up with every chunk."""
    n, g = world * 32 + 5, 16
    rng = np.random.default_rng(world)
    buckets = [rng.standard_normal(n).astype(np.float32) for _ in range(world)]
    trace = []
    ring_np.ring_all_reduce(buckets, "fp32", g, trace=trace)
    assert len(trace) == 2 * (world - 1) * world
    for phase, step, rank, sent, received_from, received in trace:
        assert received_from == (rank - 1) % world
        if phase == "reduce":
            assert sent == (rank - step - 1) % world and received == (rank - step - 2) % world
        else:
            assert sent == (rank - step) % world and received == (rank - step - 1) % world
    for rank in range(world):
        assert [t[5] for t in trace if t[0] == "reduce" and t[2] == rank][-1] == rank
        assert {t[5] for t in trace if t[0] == "gather" and t[2] == rank} | {rank} == set(range(world))


def test_the_owner_keeps_the_unquantized_mean_and_its_successor_the_quantized_one():
    world, g = 4, 16
    n = world * 64
    rng = np.random.default_rng(3)
    buckets = [rng.standard_normal(n).astype(np.float32) for _ in range(world)]
    results = ring_np.ring_all_reduce(buckets, "fp32", g)
    for owner in range(world):
        a, b = owner * 64, (owner + 1) * 64
        own = results[owner][a:b]
        codes, scales = codec_np.quantize(own, g)
        nxt = results[(owner + 1) % world][a:b]
        assert np.array_equal(nxt, codec_np.dequantize(codes, scales, 64, g, "fp32"))
        assert not np.array_equal(nxt, own)


@pytest.mark.parametrize("compact", [False, True])
@pytest.mark.parametrize("world, n, g", [(2, 64 * 6, 64), (4, 4 * 32 * 5, 32), (8, 8 * 16 * 3, 16)])
def test_ring_in_the_cuda_byte_format_returns_the_exact_mean_on_lossless_inputs(world, n, g, compact):
    """Same construction in the other payload format: a group maximum of 127 * 2^j * K is stored exactly, the
    extreme codes are +-127 and decode by (scale / 127) = 2^j * K exactly."""
    rng = np.random.default_rng(world * 77 + n)
    buckets, exact_sum = lossless_buckets(world, n, g, rng)
    codec = ring_np.CudaWireCodec(g, compact=compact)
    results = ring_np.ring_all_reduce(buckets, "fp32", g, codec=codec)
    want = (exact_sum / world).astype(np.float32)
    for rank in range(world):
        assert np.array_equal(results[rank], want), rank


def test_the_two_codecs_divide_differently_where_the_reference_does():
    """True division on the CPU codec's path, multiplication by the float32 reciprocal where the division runs
    on the device: they differ in the last bit for some inputs when W is not a power of two."""
    x = np.arange(1, 4001, dtype=np.float32)
    exact = ring_np.PortableCodec().divide(x, "fp32", 3.0)
    device = ring_np.CudaWireCodec().divide(x, "fp32", 3.0)
    assert np.array_equal(exact, (x / np.float32(3.0)).astype(np.float32))
    assert np.array_equal(device, (x * (np.float32(1.0) / np.float32(3.0))).astype(np.float32))
    assert 0 < np.count_nonzero(exact != device) < x.size
    assert np.array_equal(ring_np.PortableCodec().divide(x, "fp32", 8.0), ring_np.CudaWireCodec().divide(x, "fp32", 8.0))


# --------------------------------------------------------------------------- #
# tree
# --------------------------------------------------------------------------- #
def test_tree_edges_of_five_ranks_are_the_ones_the_reference_test_spells_out():
    """tests/cuda/test_topology_executors.py:1711-1745 names, for five ranks and root 0, the reduce edges in
    order: 4->1, 3->1, 2->0, 1->0."""
    assert ring_np.tree_edges(5, 0) == [(4, 1), (3, 1), (2, 0), (1, 0)]
    assert ring_np.tree_edges(1, 0) == []
    assert ring_np.tree_edges(2, 1) == [(0, 1)]


@pytest.mark.parametrize("world", [2, 3, 5, 8, 13])
def test_tree_reaches_every_rank_once_without_cycles_for_every_root(world):
    for root in range(world):
        edges = ring_np.tree_edges(world, root)
        parents = dict(edges)
        assert len(edges) == world - 1 and set(parents) == set(range(world)) - {root}
        for child in parents:
            seen, at = set(), child
            while at != root:
                assert at not in seen
                seen.add(at)
                at = parents[at]
        position = {rank: k for k, rank in enumerate([child for child, _ in edges])}
        for child, parent in edges:                      # a rank's children are listed before its own edge up
            if parent != root:
                assert position[child] < position[parent]
        assert all(sum(1 for _, p in edges if p == rank) <= 2 for rank in range(world))


def whole_bucket_lossless(world, n, g, rng):
    signs = rng.choice(np.array([-1.0, 1.0], dtype=np.float32), size=n)
    local = np.arange(n) // g
    groups = int(local[-1]) + 1
    base = signs * np.float32(127.0) * np.exp2(rng.integers(-12, 4, size=groups)[local]).astype(np.float32)
    factors = np.stack([rng.integers(1, 6, size=groups)[local] for _ in range(world)])
    buckets = [(base * factors[r].astype(np.float32)).astype(np.float32) for r in range(world)]
    return buckets, base.astype(np.float64) * factors.sum(axis=0)


@pytest.mark.parametrize("codec", ["portable", "cuda"])
@pytest.mark.parametrize("world, n, g, root", [(2, 64 * 3, 64, 0), (4, 32 * 9, 32, 3), (8, 16 * 21, 16, 5)])
def test_tree_all_reduce_returns_the_exact_mean_when_every_quantization_is_lossless(world, n, g, root, codec):
    rng = np.random.default_rng(world * 31 + root)
    buckets, exact_sum = whole_bucket_lossless(world, n, g, rng)
    active = ring_np.PortableCodec(g) if codec == "portable" else ring_np.CudaWireCodec(g, compact=True)
    results = ring_np.tree_all_reduce(buckets, "fp32", g, codec=active, root=root)
    want = (exact_sum / world).astype(np.float32)
    assert np.array_equal(want.astype(np.float64), exact_sum / world)
    for rank in range(world):
        assert np.array_equal(results[rank], want), rank


def test_tree_keeps_the_unquantized_mean_at_the_root_and_quantizes_once_per_level():
    world, n, g, root = 5, 16 * 40 + 3, 16, 2
    rng = np.random.default_rng(9)
    buckets = [rng.standard_normal(n).astype(np.float32) for _ in range(world)]
    results = ring_np.tree_all_reduce(buckets, "fp32", g, root=root)
    parents = dict(ring_np.tree_edges(world, root))
    for rank in range(world):
        if rank == root:
            continue
        above = results[parents[rank]]
        codes, scales = codec_np.quantize(above, g)
        assert np.array_equal(results[rank], codec_np.dequantize(codes, scales, n, g, "fp32")), rank
    first_child = next(child for child, parent in parents.items() if parent == root)
    assert not np.array_equal(results[root], results[first_child])
    exact = np.mean([b.astype(np.float64) for b in buckets], axis=0)
    peak = sum(float(np.max(np.abs(b))) for b in buckets)
    assert np.max(np.abs(results[root].astype(np.float64) - exact)) <= 3 * peak / 254 / world * world
    single = ring_np.tree_all_reduce([buckets[0]], "fp32", g)
    assert np.array_equal(single[0], buckets[0])
