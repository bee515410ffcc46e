"""CPU oracle (numpy) for the general quantize / dequantize kernels of the reference's CUDA extension.
TEST INFRASTRUCTURE ONLY: only tests, the smoke check and the benchmark's CPU-baseline leg may import it.

``ccdl_cuda_ops.quantize`` / ``inplace_quantize`` / ``dequantize`` run these kernels for every policy, and
``inplace_quantize_pack`` hands them every call without a residual whose length is a multiple of the group
size (quant_pack_kernel.cu:231,259-262).  On top of the linear 8-/4-bit format restated in ``cuda_wire_np``
they add:

* non-linear 4-bit code books ``normal``, ``uniform``, ``e3m0``, ``e2m1`` (inner.cuh:9-35,74-97,118-138):
  ``t = v / max(scale, 1e-6)``, the code is the entry nearest to ``t`` (upper neighbour only when strictly
  past the midpoint), decode is ``book[code] * scale``;
* stochastic rounding (inner.cuh:52-55,89-92): one ``curand_uniform`` per element from a Philox4x32-10
  stream whose subsequence is the group's index and whose offset is the generator's
  (quant_kernel_fp32.cuh:168-174, quant_kernel.cuh:112-120); linear codes add ``u - 0.5`` before rounding,
  code-book codes move up when ``u < (t - lower) / (upper - lower)``;
* a top-k side channel, k = 1 or 2 (quant_kernel_fp32.cuh:87-165, quant_kernel.cuh:25-106): the k largest
  magnitudes of a group travel verbatim behind the scale as ``[scale][indices][top1][top2]`` words of the
  tensor's item size, are encoded as zero, and the scale is the next largest magnitude
  (layout: quant_kernel_fp32.cuh:283-331,390-417; reader: dequant_kernel_fp32.cuh:171-216,267-330);
* the group maximum as a running ``(m > a) ? m : a`` (utils.cuh:11-14), which a NaN resets;
* for fp16/bf16 tensors a scan of each group that starts at element ``4 * ((group & 31) / (32 / (g / 4)))``
  and wraps (quant_kernel.cuh:30-32,114-116): it decides ties of the top-k search, which element a NaN
  reset sees last and which uniform an element gets.

Everything is vectorised over groups and walks the g scan positions in a Python loop, so the running
comparisons are literally the reference's.  ``cuda_wire_general_scalar.c`` restates the same kernels one
group at a time; the tests hold the two against each other, against exact rational arithmetic, against
the Philox known-answer vectors of the Random123 distribution and against closed forms of the code books; a GPU
test holds ``curand_draws`` against rocRAND's Philox device generator (documented to reproduce cuRAND's sequence).

Parity with an actual NVIDIA build is unpinned (the reference holds no payload bytes for these policies):
in particular whether nvcc contracts ``v * m + noise`` into one FMA (its default, restated here).
"""
from __future__ import annotations

import numpy as np

from .cuda_wire_np import (_ITEMSIZE, _add_in_dtype, _pack_nibbles, _swap_words, _unpack_nibbles, fma_f32, from_f32,
                           num_groups, to_f32)

_INF = np.float32(np.inf)
# inner.cuh:9-35, the literals as written there (float32 of each decimal); entry 15 is +inf.
CODE_BOOKS = {
    "normal": np.array([-1.0, -0.815410147, -0.655160150, -0.510228027, -0.375324982, -0.246951370, -0.122538030,
                        0.0, 0.122538030, 0.246951370, 0.375324982, 0.510228027, 0.655160150, 0.815410147, 1.0,
                        np.inf], dtype=np.float32),
    "uniform": np.array([-1.0, -0.85714286, -0.71428571, -0.57142857, -0.42857143, -0.28571429, -0.14285714, 0.0,
                         0.14285714, 0.28571429, 0.42857143, 0.57142857, 0.71428571, 0.85714286, 1.0, np.inf],
                        dtype=np.float32),
    "e3m0": np.array([-1.0, -0.5, -0.25, -0.125, -0.0625, -0.03125, -0.015625, 0.0, 0.015625, 0.03125, 0.0625,
                      0.125, 0.25, 0.5, 1.0, np.inf], dtype=np.float32),
    "e2m1": np.array([-1.0, -0.6666666666666666, -0.5, -0.3333333333333333, -0.25, -0.16666666666666666, -0.125,
                      0.0, 0.125, 0.16666666666666666, 0.25, 0.3333333333333333, 0.5, 0.6666666666666666, 1.0,
                      np.inf], dtype=np.float32),
}
QUANT_TYPES = ("linear",) + tuple(CODE_BOOKS)
_META_WORDS = {0: 1, 1: 3, 2: 4}       # scale | scale, indices, top1 | scale, indices, top1, top2
_UINT = {4: np.uint32, 2: np.uint16}


def payload_nbytes(numel: int, group_size: int, dtype: str, bit: int = 8, topk: int = 0) -> int:
    """gen_code_quant.py:167-178."""
    return num_groups(numel, group_size) * (group_size * bit // 8 + _ITEMSIZE[dtype] * _META_WORDS[topk])


def scan_start(group_index: np.ndarray, group_size: int, dtype: str) -> np.ndarray:
    """First element of a group's scan: 0 for fp32 tensors, bank-rotated for 16-bit ones."""
    group_index = np.asarray(group_index, dtype=np.int64)
    if dtype == "fp32":
        return np.zeros_like(group_index)
    banks = group_size // 4
    return 4 * ((group_index & 31) // (32 // banks))


# ---------------------------------------------------------------------------------------------------------
# Philox4x32-10 and the cuRAND stream built on it
# ---------------------------------------------------------------------------------------------------------
_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = 0x9E3779B9, 0xBB67AE85
_MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter, key):
    """counter: 4 uint32 arrays (x, y, z, w), key: 2 uint32 arrays -> 4 uint32 arrays."""
    c = [np.asarray(v, dtype=np.uint64) & _MASK for v in counter]
    k = [np.asarray(v, dtype=np.uint64) & _MASK for v in key]
    for round_index in range(10):
        if round_index:
            k = [(k[0] + np.uint64(_W0)) & _MASK, (k[1] + np.uint64(_W1)) & _MASK]
        p0, p1 = _M0 * c[0], _M1 * c[2]
        c = [(p1 >> np.uint64(32)) ^ c[1] ^ k[0], p1 & _MASK, (p0 >> np.uint64(32)) ^ c[3] ^ k[1], p0 & _MASK]
    return [v.astype(np.uint32) for v in c]


def curand_draws(seed: int, subsequence: np.ndarray, offset: int, count: int) -> np.ndarray:
    """The first ``count`` 32-bit outputs of ``curand_init(seed, subsequence, offset)`` for every subsequence:
    the counter's upper half is the subsequence, its lower half ``(offset + j) / 4``, and draw j is word
    ``(offset + j) % 4`` of that block."""
    subsequence = np.asarray(subsequence, dtype=np.uint64).reshape(-1)
    position = np.uint64(offset) + np.arange(count, dtype=np.uint64)
    first, last = int(position[0] >> np.uint64(2)), int(position[-1] >> np.uint64(2))
    key = [np.uint64(seed & 0xFFFFFFFF), np.uint64((seed >> 32) & 0xFFFFFFFF)]
    blocks = []
    for block in range(first, last + 1):
        counter = [np.full(subsequence.shape, block & 0xFFFFFFFF, dtype=np.uint64),
                   np.full(subsequence.shape, (block >> 32) & 0xFFFFFFFF, dtype=np.uint64),
                   subsequence & _MASK, subsequence >> np.uint64(32)]
        blocks.append(np.stack(philox4x32_10(counter, key), axis=1))            # [groups, 4]
    words = np.concatenate(blocks, axis=1)                                        # [groups, 4 * blocks]
    start = int(position[0] & np.uint64(3))
    return np.ascontiguousarray(words[:, start:start + count])


def curand_uniform(draws: np.ndarray) -> np.ndarray:
    """``x * 2^-32 + 2^-33`` in float32: the conversion of x rounds to 24 bits, the rest is exact."""
    return (draws.astype(np.float32) * np.float32(2.0 ** -32) + np.float32(2.0 ** -33)).astype(np.float32)


# ---------------------------------------------------------------------------------------------------------
# quantize
# ---------------------------------------------------------------------------------------------------------
def _gather(rows: np.ndarray, index: np.ndarray) -> np.ndarray:
    return rows[np.arange(rows.shape[0]), index]


def _scale_and_topk(rows_bits: np.ndarray, rows: np.ndarray, start: np.ndarray, dtype: str, topk: int):
    """rows: float32 values [groups, g] (modified in place: the top-k elements become 0); rows_bits: the same
    elements as stored (uint32 / uint16).  -> (stored scale bits, top1 index, top2 index, top1 bits, top2 bits)."""
    groups, g = rows.shape
    wide = dtype == "fp32"
    uint = _UINT[_ITEMSIZE[dtype]]
    sign_clear = uint(0x7FFFFFFF if wide else 0x7FFF)
    magnitude = np.abs(rows)

    def beats(a, b):          # fp32 kernels compare with >=, 16-bit kernels with __hgt
        return a >= b if wide else a > b

    top = [np.zeros(groups, dtype=np.float32) for _ in range(3)]
    top_bits = [np.zeros(groups, dtype=uint) for _ in range(3)]       # magnitude bits of top[k]
    index = [np.full(groups, -1, dtype=np.int64) for _ in range(2)]
    with np.errstate(invalid="ignore"):
        for j in range(g):
            i = (start + j) & (g - 1)
            a, a_bits = _gather(magnitude, i), _gather(rows_bits, i) & sign_clear
            if topk == 0:
                keep = top[0] > a                                     # (m > a) ? m : a
                top[0] = np.where(keep, top[0], a)
                top_bits[0] = np.where(keep, top_bits[0], a_bits)
                continue
            first = beats(a, top[0])
            second = ~first & beats(a, top[1])
            if topk == 2:
                third = ~first & ~second & beats(a, top[2])
                moved = first | second                                # the old second drops to third
                top[2] = np.where(moved, top[1], np.where(third, a, top[2]))
                top_bits[2] = np.where(moved, top_bits[1], np.where(third, a_bits, top_bits[2]))
                index[1] = np.where(first, index[0], np.where(second, i, index[1]))
            top[1] = np.where(first, top[0], np.where(second, a, top[1]))
            top_bits[1] = np.where(first, top_bits[0], np.where(second, a_bits, top_bits[1]))
            top[0] = np.where(first, a, top[0])
            top_bits[0] = np.where(first, a_bits, top_bits[0])
            index[0] = np.where(first, i, index[0])
    if topk == 0:
        return top_bits[0], None, None, None, None
    none = index[0] < 0
    if topk == 1:
        # nothing qualified: index 0, and the scale is element 1 (as stored for fp32, its magnitude for 16-bit)
        second_element = rows_bits[:, 1] if wide else rows_bits[:, 1] & sign_clear
        scale_bits = np.where(none, second_element, top_bits[1])
        index[0] = np.where(none, 0, index[0])
    else:
        lonely = ~none & (index[1] < 0)
        index[1] = np.where(none, 1, np.where(lonely, (index[0] + 1) % g, index[1]))
        index[0] = np.where(none, 0, index[0])
        scale_bits = np.where(none | lonely, uint(0), top_bits[2])
    rows_index = np.arange(groups)
    top1_bits = rows_bits[rows_index, index[0]].copy()
    rows[rows_index, index[0]] = 0.0
    top2_bits = None
    if topk == 2:
        top2_bits = rows_bits[rows_index, index[1]].copy()
        rows[rows_index, index[1]] = 0.0
    return scale_bits.astype(uint), index[0], index[1] if topk == 2 else None, top1_bits, top2_bits


def _bits_to_f32(bits: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "fp32":
        return np.ascontiguousarray(bits, dtype=np.uint32).view(np.float32)
    if dtype == "fp16":
        return np.ascontiguousarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def _stored_bits(x: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "fp32":
        return np.ascontiguousarray(x, dtype=np.float32).reshape(-1).view(np.uint32)
    if dtype == "fp16":
        return np.ascontiguousarray(x, dtype=np.float16).reshape(-1).view(np.uint16)
    return np.ascontiguousarray(x, dtype=np.uint16).reshape(-1)


def quantize(x: np.ndarray, dtype: str, group_size: int = 64, bit: int = 8, quant_type: str = "linear",
             topk: int = 0, stochastic: tuple[int, int] | None = None, compact: bool = False,
             first_group: int = 0) -> np.ndarray:
    """``stochastic`` is the generator's (seed, offset) pair, None for round-to-nearest.  ``first_group`` restates a
    window of a larger tensor: the index of the window's first group there (it fixes the 16-bit scan start and the
    Philox subsequence of every group; the appended layout of a window is the window's own)."""
    if quant_type not in QUANT_TYPES or bit not in (4, 8) or (quant_type != "linear" and bit != 4):
        raise ValueError((quant_type, bit))
    item = _ITEMSIZE[dtype]
    bits = _stored_bits(x, dtype)
    if bits.size % group_size:
        raise ValueError("input numel should be multiple of group_size")        # gen_code_quant.py:164
    groups = bits.size // group_size
    if groups == 0:
        return np.empty(0, dtype=np.uint8)
    rows_bits = bits.reshape(groups, group_size)
    rows = _bits_to_f32(bits, dtype).reshape(groups, group_size).copy()
    group_index = np.arange(groups, dtype=np.int64) + int(first_group)
    start = scan_start(group_index, group_size, dtype)
    scale_bits, index1, index2, top1_bits, top2_bits = _scale_and_topk(rows_bits, rows, start, dtype, topk)

    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        scale = _bits_to_f32(scale_bits, dtype)
        scale = np.where(scale < 1e-6, np.float32(1e-6), scale).astype(np.float32)   # a NaN scale stays NaN
        uniform = None
        if stochastic is not None:
            by_scan = curand_uniform(curand_draws(stochastic[0], group_index, stochastic[1], group_size))
            # element i of a group is visited at scan position (i - start) mod g
            position = (np.arange(group_size)[None, :] - start[:, None]) & (group_size - 1)
            uniform = np.take_along_axis(by_scan, position, axis=1)
        if quant_type == "linear":
            levels = np.float32(127.0 if bit == 8 else 7.0)
            multiplier = (np.float64(levels) / scale.astype(np.float64)).astype(np.float32)[:, None]
            if uniform is None:
                value = (rows * multiplier).astype(np.float32)
            else:
                noise = (uniform.astype(np.float64) - 0.5).astype(np.float32)
                value = fma_f32(rows, np.broadcast_to(multiplier, rows.shape), noise)
            rounded = np.rint(value)
            rounded = np.where(np.isnan(rounded), np.float32(0.0), rounded)          # __float2int_rn(NaN) = 0
            codes = np.clip(rounded, -levels, levels).astype(np.int8)
        else:
            book = CODE_BOOKS[quant_type]
            t = (rows / scale[:, None]).astype(np.float32)
            lower = np.zeros(rows.shape, dtype=np.int64)
            for mid in range(1, 15):                      # largest l in [0, 14] with not (t < book[l]); NaN -> 14
                lower += ~(t < book[mid])
            gap = (book[lower + 1] - book[lower]).astype(np.float32)
            excess = (t - book[lower]).astype(np.float32)
            if uniform is None:
                up = excess > (gap / np.float32(2.0)).astype(np.float32)
            else:
                up = uniform < (excess / gap).astype(np.float32)
            codes = (lower + up).astype(np.int8)

    if bit == 8:
        code_bytes = _swap_words(codes.view(np.uint8).reshape(-1), item).reshape(groups, group_size)
    else:
        code_bytes = _pack_nibbles(codes.reshape(-1), item).reshape(groups, group_size // 2)
    uint = _UINT[item]
    meta = [scale_bits.astype(uint)]
    if topk == 1:
        meta += [index1.astype(uint), top1_bits.astype(uint)]
    elif topk == 2:
        meta += [(index1 | (index2 << 8)).astype(uint), top1_bits.astype(uint), top2_bits.astype(uint)]
    meta_bytes = np.ascontiguousarray(np.stack(meta, axis=1)).view(np.uint8).reshape(groups, -1)
    if compact:
        return np.ascontiguousarray(np.concatenate([code_bytes, meta_bytes], axis=1)).reshape(-1)
    return np.concatenate([code_bytes.reshape(-1), meta_bytes.reshape(-1)])


def quantize_pack(x: np.ndarray, dtype: str, group_size: int = 64, compact: bool = True,
                  residual: np.ndarray | None = None, bit: int = 8) -> np.ndarray:
    """What ``inplace_quantize_pack`` writes for a plain linear policy (quant_pack_kernel.cu:231,259-275): whole
    groups without a residual go to the general kernels (running maximum, a NaN resets it), everything else to
    the fused pack kernel (``fmaxf``, NaNs skipped).  The two differ only on groups that hold a NaN."""
    from .cuda_wire_np import quantize as pack_kernel

    n = np.asarray(x).size
    if residual is None and n % group_size == 0:
        return quantize(x, dtype, group_size, bit, "linear", 0, None, compact)
    return pack_kernel(x, dtype, group_size, compact, residual, bit)


# ---------------------------------------------------------------------------------------------------------
# dequantize
# ---------------------------------------------------------------------------------------------------------
def split(payload: np.ndarray, numel: int, dtype: str, group_size: int, bit: int, topk: int, compact: bool):
    """-> (codes [groups, g] as unsigned nibbles / signed bytes, meta words [groups, 1|3|4] as stored)."""
    item = _ITEMSIZE[dtype]
    groups = numel // group_size
    per_group = group_size * bit // 8
    words = _META_WORDS[topk]
    payload = np.ascontiguousarray(payload, dtype=np.uint8).reshape(-1)
    assert payload.size == groups * (per_group + words * item)
    if compact:
        table = payload.reshape(groups, per_group + words * item)
        code_bytes = np.ascontiguousarray(table[:, :per_group]).reshape(-1)
        meta_bytes = np.ascontiguousarray(table[:, per_group:]).reshape(-1)
    else:
        code_bytes = payload[: groups * per_group]
        meta_bytes = np.ascontiguousarray(payload[groups * per_group:])
    if bit == 8:
        codes = _swap_words(code_bytes, item).view(np.int8)
    else:
        codes = _unpack_nibbles(code_bytes, item)
    return codes.reshape(groups, group_size), meta_bytes.view(_UINT[item]).reshape(groups, words)


def dequantize(payload: np.ndarray, numel: int, dtype: str, group_size: int = 64, bit: int = 8,
               quant_type: str = "linear", topk: int = 0, compact: bool = False, reduce_op: str = "none",
               out: np.ndarray | None = None) -> np.ndarray:
    if numel % group_size:
        raise ValueError("numel should be multiple of group_size")
    codes, meta = split(payload, numel, dtype, group_size, bit, topk, compact)
    groups = codes.shape[0]
    with np.errstate(invalid="ignore", over="ignore"):
        scale = _bits_to_f32(meta[:, 0], dtype)
        if quant_type == "linear":
            step = (scale.astype(np.float64) / (127.0 if bit == 8 else 7.0)).astype(np.float32)
            values = (codes.astype(np.float32) * step[:, None]).astype(np.float32)
        else:
            book = CODE_BOOKS[quant_type]
            values = (book[codes.astype(np.int64) & 15] * scale[:, None]).astype(np.float32)
    stored = _stored_bits(from_f32(values.reshape(-1), dtype), dtype).reshape(groups, group_size).copy()
    rows_index = np.arange(groups)
    if topk >= 1:
        stored[rows_index, (meta[:, 1] & 0xFF).astype(np.int64)] = meta[:, 2]
    if topk == 2:
        stored[rows_index, ((meta[:, 1] >> 8) & 0xFF).astype(np.int64)] = meta[:, 3]
    view = {"fp32": np.float32, "fp16": np.float16, "bf16": np.uint16}[dtype]
    value = stored.reshape(-1).view(view)
    if reduce_op == "none":
        return value
    assert out is not None
    if reduce_op == "sum":
        return _add_in_dtype(out, value, dtype)
    old, new = to_f32(out, dtype).reshape(-1), to_f32(value, dtype)
    pick_old = old > new if reduce_op == "max" else ~(old > new)       # utils.cuh:11-14
    return np.where(pick_old, np.asarray(out).reshape(-1), value)
