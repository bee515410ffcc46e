// The policies of the reference's CUDA extension beyond plain linear codes, in its payload format:
// non-linear 4-bit code books, stochastic rounding, the top-k side channel and the group maximum that
// a NaN resets (ccdl_comm/csrc/quantization/quant_kernel_fp32.cuh, quant_kernel.cuh, inner.cuh,
// dequant_kernel_fp32.cuh, dequant_kernel.cuh).  ccdl_cuda_ops.quantize / dequantize run these
// kernels for every policy; inputs are whole groups (gen_code_quant.py:164).
//
// Payload of a group, in words of the tensor's item size (quant_kernel_fp32.cuh:283-331,390-417):
//   [code words][scale]                                   top-k 0
//   [code words][scale][index][top1]                      top-k 1
//   [code words][scale][index1 | index2 << 8][top1][top2] top-k 2
// with the metadata behind each group's codes (compact) or behind all codes.  The top-k elements are
// stored as they are, encoded as zero, and the scale is the next largest magnitude.
//
// The reference walks a group with one thread, element by element: fp32 groups from element 0,
// fp16/bf16 groups from element 4 * ((group & 31) / (32 / (G / 4))) with wrap-around.  That order
// decides (a) which elements a NaN hides from the running maximum `(m > a) ? m : a`, (b) ties of the
// top-k search (fp32 compares with >=: the later element wins and zeros qualify; 16-bit compares
// with >: the earlier element of the scan wins and zeros do not), (c) which draw of the group's
// Philox stream an element receives.  Here a group lies across G/VEC lanes of a DPP row as in the
// other kernels, and each of the three is restated in an order-free form: (a) the maximum over the
// scan positions behind the last NaN, (b) the three largest keys (magnitude bits, tie-break rank),
// merged across the row, (c) Philox in counter mode - draw j of group s is word (offset + j) % 4
// of block (offset + j) / 4 of subsequence s, so a lane computes the blocks of its own elements.
#include "code_book_cells.h"
#include "device_utils.h"
#include "launch.h"
#include "wire_common.h"

namespace lbc {
namespace {

// inner.cuh:9-35, and the one-lookup form of the encoder built from them at compile time
__constant__ book_cells::Books kCodeBooks = book_cells::kBookSet;
__constant__ book_cells::Tables kBookCells = book_cells::kTables;

// Philox4x32-10: one block of four 32-bit words.  A round is two 32x32->64 multiplies and two three-way
// exclusive-ors; gfx950 has the latter as one instruction (v_bitop3_b32 with the truth table 0x96), which the
// compiler does not choose by itself for `a ^ b ^ c`.
__device__ __forceinline__ uint32_t xor3(uint32_t x, uint32_t y, uint32_t z) {
    return __builtin_amdgcn_bitop3_b32(x, y, z, 0x96);
}

__device__ __forceinline__ void philox_block(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1,
                                             uint32_t (&out)[4]) {
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        if (round) {
            k0 += 0x9E3779B9u;
            k1 += 0xBB67AE85u;
        }
        const uint64_t p0 = static_cast<uint64_t>(0xD2511F53u) * c0, p1 = static_cast<uint64_t>(0xCD9E8D57u) * c2;
        const uint32_t n0 = xor3(static_cast<uint32_t>(p1 >> 32), c1, k0), n2 = xor3(static_cast<uint32_t>(p0 >> 32), c3, k1);
        c0 = n0;
        c1 = static_cast<uint32_t>(p1);
        c2 = n2;
        c3 = static_cast<uint32_t>(p0);
    }
    out[0] = c0;
    out[1] = c1;
    out[2] = c2;
    out[3] = c3;
}

// Each wavefront keeps its own copy of the code book in LDS: written and read by the same wavefront, whose LDS
// operations execute in order, so no workgroup barrier stands between the first loads and the arithmetic.
__device__ __forceinline__ const float *wave_code_book(int kind, int lane) {
    __shared__ float books[kWavesPerBlock][16];
    float *book = books[threadIdx.x >> 6];
    if (kind != 0) {
        if (lane < 16) book[lane] = kCodeBooks.value[kind - 1][lane];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    return book;
}

// The workgroup's copy of a book's cell table (code_book_cells.h) in LDS.  Every wavefront of the workgroup must
// come here: the copy ends in a workgroup barrier.
__device__ __forceinline__ const book_cells::Cell *block_book_cells(int kind) {
    __shared__ book_cells::Cell cells[book_cells::kCells];
    static_assert(book_cells::kCells <= kBlock + 1, "one table entry per thread, and one more");
    const book_cells::Cell *table = kBookCells.book[kind - 1].cell;
    cells[threadIdx.x] = table[threadIdx.x];
    if (threadIdx.x == 0) cells[kBlock] = table[kBlock];
    __syncthreads();
    return cells;
}

__device__ __forceinline__ int meta_words_of(int topk) { return topk == 0 ? 1 : topk + 2; }

// ---------------------------------------------------------------------------------------------
// quantize: a wavefront works on tiles of 64 * EL elements (64 lanes x 32 bytes of the tensor, 16 for one policy)
// ---------------------------------------------------------------------------------------------
// Elements per lane: 32 bytes of the tensor, twice what the other kernels of this format give a lane.  What a
// policy costs per group - addresses, the NaN rule of the running maximum, the outlier searches, the division behind
// the scale - is spread over twice the elements, and a group's reductions cross half the lanes.  These kernels are
// bound by instruction work and latency, not by memory, so that is what counts (26.2 M elements, 16 against 32 bytes a
// lane: see the measurements at launch_general_quant_g).
template <typename T> constexpr int general_quant_elems() { return 32 / static_cast<int>(sizeof(T)); }

// The EL 4-bit codes of one lane -> its 32-bit words.  Four codes make one 16-bit unit with the first code on top; a
// 16-bit tensor's word holds two units, low half first, an fp32 tensor's word holds elements 0-3 in its upper half.
template <typename T, int EL>
__device__ __forceinline__ void pack_nibbles(const int (&c)[EL], uint32_t (&words)[EL / 8]) {
#pragma unroll
    for (int k = 0; k < EL / 8; ++k) {
        uint32_t unit[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            unit[h] = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) unit[h] |= (static_cast<uint32_t>(c[8 * k + 4 * h + i]) & 0xFu) << (12 - 4 * i);
        }
        words[k] = sizeof(T) == 4 ? (unit[0] << 16) | unit[1] : unit[0] | (unit[1] << 16);
    }
}

__device__ __forceinline__ uint32_t umed3(uint32_t x, uint32_t y, uint32_t z) {
    uint32_t m;
    asm("v_med3_u32 %0, %1, %2, %3" : "=v"(m) : "v"(x), "v"(y), "v"(z));
    return m;
}

// first >= second >= third are the three largest keys a lane knows (0 = none; nonzero keys are unique inside a
// group).  Afterwards every lane of the group's LANES adjacent lanes holds the three largest of the group.  With
// p, q = max, min of the two firsts, r, s = max, min of the seconds and t = max of the thirds, the union's first is
// p, its second max(q, r) and its third max(min(q, r), s, t).  row_half_mirror and row_mirror act as xor 4 / xor 8
// because the lanes they pair within a quad (half) already agree.
template <int CTRL> __device__ __forceinline__ void merge_top3_step(uint32_t &first, uint32_t &second, uint32_t &third) {
    auto partner = [](uint32_t v) {
        return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xF, 0xF, true));
    };
    const uint32_t f = partner(first), g = partner(second), h = partner(third);
    const uint32_t p = first > f ? first : f, q = first > f ? f : first;
    const uint32_t r = second > g ? second : g, s = second > g ? g : second;
    const uint32_t t = third > h ? third : h;
    const uint32_t low = q < r ? q : r;
    first = p;
    second = q > r ? q : r;
    third = low > s ? (low > t ? low : t) : (s > t ? s : t);
}

template <int LANES> __device__ __forceinline__ void merge_top3(uint32_t &first, uint32_t &second, uint32_t &third) {
    static_assert(LANES == 1 || LANES == 2 || LANES == 4 || LANES == 8 || LANES == 16, "row-sized groups only");
    if constexpr (LANES >= 2) merge_top3_step<0xB1>(first, second, third);    // quad_perm [1,0,3,2]
    if constexpr (LANES >= 4) merge_top3_step<0x4E>(first, second, third);    // quad_perm [2,3,0,1]
    if constexpr (LANES >= 8) merge_top3_step<0x141>(first, second, third);   // row_half_mirror
    if constexpr (LANES >= 16) merge_top3_step<0x140>(first, second, third);  // row_mirror
}

// FIXED names what the launch knows about the policy at compile time, so that the code of the other policies
// is not part of the kernel: bit 0 "no outlier channel", bit 1 "round to nearest", bit 2 "linear codes", bit 3
// "stochastic rounding" (13: plain linear codes rounded stochastically, 12: the same with outliers, 9: a code book
// with stochastic rounding).  0 is the kernel for every policy.
// EL: elements per lane, a multiple of 8 that divides G.  TILES: tiles of 64 * EL elements a wavefront owns, all of
// them asked for before the first is encoded.
template <typename T, int G, int BIT, int FIXED, int EL, int TILES>
__global__ __launch_bounds__(kBlock) void wire_general_quant_kernel(const WireGeneralQuantArgs a) {
    const int topk = (FIXED & 1) ? 0 : a.topk;
    const bool stochastic = (FIXED & 2) ? false : ((FIXED & 8) ? true : a.stochastic != 0);
    const int kind = (FIXED & 4) ? 0 : a.kind;
    using W = wire<T, BIT>;
    using RB = raw_bits<T>;
    using Raw = typename RB::type;
    constexpr int VEC = EL, LPG = G / VEC, ITEM = sizeof(T), CB = G * BIT / 8, WORDS = EL * BIT / 32;
    constexpr bool WIDE = ITEM == 4;
    static_assert(EL % 8 == 0 && EL % W::VEC == 0 && G % EL == 0 && LPG <= 16, "a group lies in 1..16 lanes of one DPP row");

    const int lane = threadIdx.x & (kWave - 1);
    const int meta_bytes = meta_words_of(topk) * ITEM;
    const int64_t groups = a.numel / G;
    constexpr int TILE = kWave * EL;
    const int64_t first = (static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6)) * (TILES * TILE);

    // all of the wavefront's elements are asked for before anything else
    Raw raws[TILES][VEC];
#pragma unroll
    for (int tile = 0; tile < TILES; ++tile) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) raws[tile][i] = 0;
        const int64_t e0 = first + tile * TILE + lane * VEC;
        // numel is a multiple of G: dead lanes form whole dead groups.  Instruction-bound: a cache hint only costs.
        if (e0 < a.numel) {
#pragma unroll
            for (int part = 0; part < EL / W::VEC; ++part) {
                Raw piece[W::VEC];
                load_elems<Raw, W::VEC, kPlain>(static_cast<const Raw *>(a.x) + e0 + part * W::VEC, piece);
#pragma unroll
                for (int i = 0; i < W::VEC; ++i) raws[tile][part * W::VEC + i] = piece[i];
            }
        }
    }
    // After the loads were issued: the waits of the tables cover theirs.  The cell table pays for its copy and its
    // barrier from eight elements a lane on.
    const bool by_cells = kind != 0 && !stochastic;   // uniform over the grid
    const book_cells::Cell *cells = by_cells ? block_book_cells(kind) : nullptr;
    if (first >= a.numel) return;   // wavefront-uniform, behind the workgroup's barrier
    const float *book = wave_code_book(kind, lane);

    auto encode_tile = [&](const int64_t tile_first, const Raw (&raw)[VEC]) __attribute__((always_inline)) {
        const int64_t e0 = tile_first + lane * VEC;
        const bool live = e0 < a.numel;
        const int64_t group = e0 / G;
        const int k0 = static_cast<int>(e0 - group * G);
        const int start = scan_start<T, G>(group);
        // The draws depend on the element's place only: they are computed while its value is still on its way.
        float uniform[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) uniform[i] = 0.0f;
        if (stochastic) {
            const uint32_t key0 = static_cast<uint32_t>(a.seed), key1 = static_cast<uint32_t>(a.seed >> 32);
            const uint32_t sub0 = static_cast<uint32_t>(group), sub1 = static_cast<uint32_t>(static_cast<uint64_t>(group) >> 32);
            const int phase = static_cast<int>(a.offset & 3);
            // curand_uniform, (0, 1]: x * 2^-32 + 2^-33.  The product is exact, so the fused form rounds as the two steps do.
            auto to_uniform = [](uint32_t x) { return __builtin_fmaf(static_cast<float>(x), 0x1p-32f, 0x1p-33f); };
            uint64_t block[VEC / 4];
#pragma unroll
            for (int q = 0; q < VEC / 4; ++q)
                block[q] = (a.offset + static_cast<uint64_t>((k0 + 4 * q - start) & (G - 1))) >> 2;   // positions are multiples of 4
            uint32_t lo[VEC / 4][4];
#pragma unroll
            for (int q = 0; q < VEC / 4; ++q)
                philox_block(static_cast<uint32_t>(block[q]), static_cast<uint32_t>(block[q] >> 32), sub0, sub1, key0, key1, lo[q]);
            if (phase == 0) {   // uniform; the offsets torch hands out are multiples of four: one block a quad
#pragma unroll
                for (int q = 0; q < VEC / 4; ++q)
#pragma unroll
                    for (int e = 0; e < 4; ++e) uniform[4 * q + e] = to_uniform(lo[q][e]);
            } else {            // a quad's draws lie across two blocks
#pragma unroll
                for (int q = 0; q < VEC / 4; ++q) {
                    uint32_t hi[4];
                    philox_block(static_cast<uint32_t>(block[q] + 1), static_cast<uint32_t>((block[q] + 1) >> 32), sub0, sub1,
                                 key0, key1, hi);
                    const uint32_t w[8] = {lo[q][0], lo[q][1], lo[q][2], lo[q][3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        uniform[4 * q + e] = to_uniform(phase == 1 ? w[e + 1] : (phase == 2 ? w[e + 2] : w[e + 3]));
                }
            }
        }

        float v[VEC];
        uint32_t mag[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            v[i] = value_of<T>(raw[i]);
            mag[i] = raw[i] & RB::ABS;
        }

        uint8_t *group_codes = a.payload + (a.compact ? group * (CB + meta_bytes) : group * CB);
        uint8_t *group_meta = a.compact ? group_codes + CB : a.payload + groups * CB + group * meta_bytes;

        uint32_t scale_raw;
        Raw meta[4] = {0, 0, 0, 0};   // [scale][indices][top1][top2]
        bool any_nan = true;   // "not known": the outlier path does not look
        if (topk == 0) {
            scale_raw = running_max_raw<T, G, VEC>(mag, k0, start, &any_nan);
        } else {
            // The three largest candidates of the group, a candidate's key being its magnitude and a tie-break rank
            // (1..G, unique inside a group; the larger rank wins).
            uint32_t best_key[3] = {0, 0, 0}, best_rank[2] = {0, 0};              // magnitude + 1, rank
            if constexpr (WIDE) {
                // Three rounds of "largest remaining candidate": the group maximum of the magnitude keys, then, among
                // the elements that hold it, the maximum of the ranks.
                uint32_t key[VEC], rank[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    rank[i] = static_cast<uint32_t>(k0 + i + 1);
                    key[i] = mag[i] <= RB::INF ? mag[i] + 1 : 0;                  // 0 stands for "none"
                }
#pragma unroll
                for (int round = 0; round < 3; ++round) {
                    if (round == 2 && topk == 1) break;                         // uniform
                    uint32_t m = 0;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) m = key[i] > m ? key[i] : m;
                    m = group_max_bits<LPG>(m);
                    best_key[round] = m;
                    if (round == 2) break;
                    uint32_t r = 0;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) r = (key[i] == m && rank[i] > r) ? rank[i] : r;
                    r = group_max_bits<LPG>(r);
                    r = m == 0 ? 0 : r;
                    best_rank[round] = r;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) key[i] = rank[i] == r ? 0 : key[i];   // taken (r = 0 matches nobody)
                }
            } else {
                // A 16-bit magnitude and its rank share one 32-bit key, (magnitude << 7) + rank, unique inside the
                // group.  A lane keeps the three largest of its own keys in order (three instructions an element), and
                // the group's lanes merge their triples over the DPP butterfly (eight instructions a step): no rounds
                // over the elements.  Zeros are no candidates: their keys are below 128, under every candidate's, and
                // are dropped from the result.  NaNs are no candidates either and their keys are above every
                // candidate's: the first pass does not look for them, and when one tops any group of the wavefront
                // (rare) the pass is repeated with every element checked.  Scan positions do not wrap inside four
                // adjacent elements (a lane's first element and the scan's start are multiples of four).
                constexpr uint32_t kBelow = 128, kAbove = (RB::INF << 7) + G;
                uint32_t largest, runner_up, bronze;
                auto search = [&](const bool checked) __attribute__((always_inline)) {
                    largest = runner_up = bronze = 0;
                    const uint32_t p0 = static_cast<uint32_t>(k0 - start) & (G - 1);
#pragma unroll
                    for (int q = 0; q < VEC / 4; ++q) {
                        const uint32_t rank0 = G - ((p0 + 4 * q) & (G - 1));      // rank = G - scan position
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const int i = 4 * q + j;
                            uint32_t key = (mag[i] << 7) + (rank0 - j);
                            if (checked) key = (mag[i] - 1u) < RB::INF ? key : 0;
                            bronze = umed3(runner_up, bronze, key);
                            runner_up = umed3(largest, runner_up, key);
                            largest = key > largest ? key : largest;
                        }
                    }
                    merge_top3<LPG>(largest, runner_up, bronze);
                };
                search(false);
                if (__ballot(largest > kAbove) != 0) search(true);   // wavefront-uniform
                largest = largest < kBelow ? 0 : largest;
                runner_up = runner_up < kBelow ? 0 : runner_up;
                bronze = bronze < kBelow ? 0 : bronze;
                const uint32_t found[3] = {largest, runner_up, bronze};
#pragma unroll
                for (int round = 0; round < 3; ++round) {   // rank 1..G <= 64 never carries into the magnitude
                    best_key[round] = found[round] == 0 ? 0 : ((found[round] - 1) >> 7) + 1;
                    if (round < 2) best_rank[round] = found[round] == 0 ? 0 : ((found[round] - 1) & 0x7Fu) + 1;
                }
            }
            auto index_of = [&](uint32_t r) {
                return WIDE ? static_cast<int>(r) - 1 : ((G - static_cast<int>(r)) + start) & (G - 1);
            };
            const bool none = best_key[0] == 0;
            const int index1 = none ? 0 : index_of(best_rank[0]);
            int index2 = -1;
            if (topk == 1) {
                // nothing comparable: the reference falls back to element 1 (as stored for fp32, its magnitude otherwise)
                const uint32_t element1 = WIDE ? static_cast<uint32_t>(raw[1]) : mag[1];
                const uint32_t fallback = static_cast<uint32_t>(__shfl(static_cast<int>(element1), lane & ~(LPG - 1)));
                scale_raw = none ? fallback : (best_key[1] == 0 ? 0u : best_key[1] - 1);
            } else {
                const bool lonely = !none && best_key[1] == 0;
                index2 = none ? 1 : (lonely ? ((index1 + 1) & (G - 1)) : index_of(best_rank[1]));
                scale_raw = (none || lonely || best_key[2] == 0) ? 0u : best_key[2] - 1;
            }
#pragma unroll
            for (int i = 0; i < VEC; ++i)
                if (k0 + i == index1 || k0 + i == index2) v[i] = 0.0f;
            // The outliers travel as they are stored.  The group's first lane fetches them from the tensor once more
            // (its wavefront has just read those lines) instead of every lane selecting among its elements; the
            // metadata words leave together at the end of the tile, when the values have long arrived.
            meta[1] = static_cast<Raw>(topk == 1 ? index1 : (index1 | (index2 << 8)));
            if (live && k0 == 0) {
                const Raw *members = static_cast<const Raw *>(a.x) + group * G;
                meta[2] = members[index1];
                if (topk == 2) meta[3] = members[index2];
            }
        }
        meta[0] = static_cast<Raw>(scale_raw);

        float scale = value_of<T>(scale_raw);
        scale = scale < 1.0e-6f ? 1.0e-6f : scale;   // a NaN scale stays NaN and encodes every element as 0

        int c[VEC];
        if (kind == 0) {
            const float multiplier = W::LEVELS / scale;
            constexpr int L = static_cast<int>(W::LEVELS);
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                // nvcc contracts v * m + noise into one FMA; without noise the product is rounded alone
                const float t = stochastic ? __builtin_fmaf(v[i], multiplier, uniform[i] - 0.5f) : v[i] * multiplier;
                const int r = cvt_i32(__builtin_rintf(t));
                c[i] = r < -L ? -L : (r > L ? L : r);
            }
        } else {
            // t = v / scale, the IEEE quotient.  A lane's elements share the divisor, so the reciprocal part of the
            // division is done once: v_rcp_f32 and one Newton step, then per element the product and two corrections.
            // These are the very operations the compiler emits for `v / scale`, minus its operand scaling and
            // special-case fix-up (v_div_scale / v_div_fmas / v_div_fixup), which change nothing while the divisor
            // lies in [2^-60, 2^60], |v| <= scale, and the dividend is not so small (below 2^-103) that the division
            // would rescale it.  The scale is at least 1e-6 here, so such a dividend means a quotient below 2^-80, and a
            // quotient below 2^-30 encodes as the book's zero whatever its last bits are: it is closer to that entry
            // than the rounding error of the comparisons with its neighbours.  A wavefront with any other divisor,
            // or with an element above its scale (only a group that holds a NaN has one) or not a number, takes the
            // division.  tests/native/quotient_check.hip compares the two forms on the device.
            float t[VEC];
            const uint32_t scale_exponent = (as_u32(scale) >> 23) & 0xFFu;
            bool unusual = scale_exponent < 127u - 60u || scale_exponent > 127u + 60u;
            // Without outliers the scale is the group's largest magnitude unless a NaN reset the running maximum, and
            // the wavefront is known to hold no NaN: no element needs to be looked at.
            if (any_nan) {   // wavefront-uniform
#pragma unroll
                for (int i = 0; i < VEC; ++i) unusual |= !(__builtin_fabsf(v[i]) <= scale);
            }
            const bool usual = __ballot(unusual) == 0;   // wavefront-uniform
            if (usual) {
                float reciprocal = __builtin_amdgcn_rcpf(scale);
                reciprocal = __builtin_fmaf(__builtin_fmaf(-scale, reciprocal, 1.0f), reciprocal, reciprocal);
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    float q = v[i] * reciprocal;
                    q = __builtin_fmaf(__builtin_fmaf(-scale, q, v[i]), reciprocal, q);
                    t[i] = __builtin_fmaf(__builtin_fmaf(-scale, q, v[i]), reciprocal, q);
                }
            } else {
#pragma unroll
                for (int i = 0; i < VEC; ++i) t[i] = v[i] / scale;
            }
            if (usual && by_cells) {
                // Every t is a number in [-1, 1]: search and rounding are one table lookup (code_book_cells.h).
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const book_cells::Cell cell = cells[static_cast<uint32_t>(__builtin_fmaf(t[i], 128.0f, 128.0f))];
                    c[i] = static_cast<int>(cell.base) + (t[i] >= cell.threshold ? 1 : 0);
                }
            } else {
            // The largest entry in [0, 14] with not (t < book[entry]); a NaN ends at 14.  Four halving steps, each
            // over all of the lane's elements so that their LDS reads are in flight together; positions are kept as
            // byte offsets into the book.
            const char *book_bytes = reinterpret_cast<const char *>(book);
            int at[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) at[i] = 0;
#pragma unroll
            for (int step = 8 * 4; step >= 4; step >>= 1) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const int mid = at[i] + step;
                    const float entry = *reinterpret_cast<const float *>(book_bytes + mid);
                    at[i] = (mid < 15 * 4 && !(t[i] < entry)) ? mid : at[i];
                }
            }
            float excess[VEC], gap[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                const float low = *reinterpret_cast<const float *>(book_bytes + at[i]);
                gap[i] = *reinterpret_cast<const float *>(book_bytes + at[i] + 4) - low;
                excess[i] = t[i] - low;
                c[i] = at[i] >> 2;
            }
            if (stochastic) {   // uniform: the second division only runs when it is needed
#pragma unroll
                for (int i = 0; i < VEC; ++i) c[i] += uniform[i] < excess[i] / gap[i] ? 1 : 0;
            } else {
#pragma unroll
                for (int i = 0; i < VEC; ++i) c[i] += excess[i] > gap[i] * 0.5f ? 1 : 0;
            }
            }
        }
        if (live) {
            uint32_t words[WORDS];
            if constexpr (BIT == 8) pack_codes<T, 8, VEC, WORDS>(c, words);
            else pack_nibbles<T, EL>(c, words);
            store_words<WORDS, ITEM, kPlain>(group_codes + k0 * BIT / 8, words);
        }
        if (live && k0 == 0) {
            Raw *words = reinterpret_cast<Raw *>(group_meta);
            if (topk == 2) {
                store_elems<Raw, 4, kPlain>(words, meta);
            } else if (topk == 1) {
                const Raw pair[2] = {meta[0], meta[1]};
                store_elems<Raw, 2, kPlain>(words, pair);
                words[2] = meta[2];
            } else {
                words[0] = meta[0];
            }
        }
    };
#pragma unroll
    for (int tile = 0; tile < TILES; ++tile) {
        const int64_t tile_first = first + tile * TILE;
        if (tile_first >= a.numel) return;   // wavefront-uniform
        encode_tile(tile_first, raws[tile]);
    }
}

// ---------------------------------------------------------------------------------------------
// dequantize (optionally combined into `out`)
// ---------------------------------------------------------------------------------------------
template <typename T, int G, int BIT>
__global__ __launch_bounds__(kBlock) void wire_general_decode_kernel(const WireGeneralDecodeArgs a) {
    using W = wire<T, BIT>;
    using Raw = typename raw_bits<T>::type;
    constexpr int VEC = W::VEC, ITEM = sizeof(T), CB = G * BIT / 8;

    const int lane = threadIdx.x & (kWave - 1);
    const int meta_bytes = meta_words_of(a.topk) * ITEM;
    const int64_t groups = a.numel / G;
    const int64_t tile_first = (static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6)) * W::TILE;
    if (tile_first >= a.numel) return;   // wavefront-uniform
    const int64_t e0 = tile_first + lane * VEC;
    const bool live = e0 < a.numel;      // dead lanes read group 0 and store nothing
    const int64_t group = live ? e0 / G : 0;
    const int k0 = live ? static_cast<int>(e0 - group * G) : 0;
    const uint8_t *group_codes = a.payload + (a.compact ? group * (CB + meta_bytes) : group * CB);
    const uint8_t *group_meta = a.compact ? group_codes + CB : a.payload + groups * CB + group * meta_bytes;

    uint32_t words[W::WORDS];
    load_piece<T, BIT, kPlain, W::WORDS>(group_codes + piece_offset<T, BIT>(k0), words);
    // the group's metadata words [scale][indices][top1][top2], fetched together with the codes
    Raw meta[4] = {0, 0, 0, 0};
    if (a.topk == 2) {
        load_elems<Raw, 4, kPlain>(reinterpret_cast<const Raw *>(group_meta), meta);
    } else if (a.topk == 1) {
        Raw pair[2];
        load_elems<Raw, 2, kPlain>(reinterpret_cast<const Raw *>(group_meta), pair);
        meta[0] = pair[0];
        meta[1] = pair[1];
        meta[2] = *reinterpret_cast<const Raw *>(group_meta + 2 * ITEM);
    } else {
        meta[0] = *reinterpret_cast<const Raw *>(group_meta);
    }
    const float scale = value_of<T>(meta[0]);
    const float *book = wave_code_book(a.kind, lane);   // after the loads were issued: its wait covers theirs
    const float step = a.kind == 0 ? step_of<BIT>(scale) : scale;

    Raw decoded[VEC];
    if (BIT == 4 && a.kind != 0) {   // uniform: the code's four bits, as they are, index the book
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int top = 16 - 16 * (i / 4) + 4 * (i % 4);   // left shift that puts the nibble on top, as in unpack_code
            decoded[i] = static_cast<Raw>(raw_from<T>(book[(words[0] << top) >> 28] * step));
        }
    } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i)
            decoded[i] = static_cast<Raw>(raw_from<T>(unpack_code<T, BIT, W::WORDS>(words, i) * step));
    }
    if (a.topk >= 1) {
        const uint32_t indices = meta[1];
        const int index1 = static_cast<int>(indices & 0xFFu);
        const int index2 = a.topk == 2 ? static_cast<int>((indices >> 8) & 0xFFu) : -1;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            if (k0 + i == index1) decoded[i] = meta[2];
            if (k0 + i == index2) decoded[i] = meta[3];   // written second, as in the reference
        }
    }
    if (!live) return;
    Raw *out = static_cast<Raw *>(a.out) + e0;
    if (a.op != 0) {
        Raw old[VEC];
        load_elems<Raw, VEC, kNonTemporal>(out, old);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const float o = value_of<T>(old[i]), d = value_of<T>(decoded[i]);
            if (a.op == 1) decoded[i] = static_cast<Raw>(raw_from<T>(add_in<T>(o, d)));
            else if (a.op == 2) decoded[i] = o > d ? old[i] : decoded[i];
            else decoded[i] = o > d ? decoded[i] : old[i];
        }
    }
    // The decoded tensor is the large stream of this kernel and nothing here reads it again: with the non-temporal
    // hint the decode of 26.2 M fp32 elements takes 19.9 instead of 30.2 us (top-2), 18.0 instead of 31.1 us (code book).
    store_elems<Raw, VEC, kNonTemporal>(out, decoded);
}

template <typename T, int G, int BIT, int FIXED, int EL, int TILES = 1>
hipError_t launch_general_quant_as(const WireGeneralQuantArgs &a, hipStream_t stream) {
    const int64_t tile = static_cast<int64_t>(kWave) * EL * kWavesPerBlock * TILES;
    const int64_t blocks = (a.numel + tile - 1) / tile;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((wire_general_quant_kernel<T, G, BIT, FIXED, EL, TILES>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0,
                       stream, a);
    return hipGetLastError();
}

template <typename T, int G>
hipError_t launch_general_quant_g(int bit, const WireGeneralQuantArgs &a, hipStream_t stream) {
    // Each common policy runs a kernel without the code of the others (26.2 M fp32 elements: top-2 30.8 instead of
    // 32.3 us, a code book 30.0 instead of 31.7 us).  Stochastic rounding of plain linear codes gains most: in the
    // kernel for every policy it holds 126 vector registers for sixteen 16-bit elements a lane (four wavefronts a
    // SIMD), on its own 65 (seven): 26.2 M bf16 elements 17.0 instead of 20.4 us, fp32 23.7 instead of 24.2 us.
    // With outliers 32.4 / 26.8 instead of 35.3 / 28.5 us (fp32 / bf16), with a code book 36.5 / 34.5 instead of
    // 40.8 / 38.8 us.
    //
    // 32 bytes a lane against 16 (26.2 M elements, group 64, us): fp32 top-2 27.4 / 30.5, stochastic 24.3 / 26.6,
    // a code book 25.5 / 27.9; bf16 top-2 22.1 / 23.3, stochastic 21.5 / 22.6, a code book through the cell table
    // 19.8 / 19.3 - the one case that keeps 16 bytes, and the one case that gains from two such tiles a wavefront,
    // both asked for before either is encoded (18.2 against 19.4 us; the others lose 8-20 % with two tiles).
    constexpr int WIDE = general_quant_elems<T>() <= G ? general_quant_elems<T>() : G;
    constexpr int CELLS = sizeof(T) == 4 ? WIDE : 8, CELL_TILES = sizeof(T) == 4 ? 1 : 2;
    const int fixed = a.stochastic ? 0 : ((a.topk == 0 ? 1 : 0) | 2 | (a.kind == 0 ? 4 : 0));
    if (bit != 8 && bit != 4) return hipErrorNotSupported;
    if (bit == 8 && a.kind != 0) return hipErrorNotSupported;   // eight bits: linear codes only
    if (bit == 8) {
        if (a.stochastic && a.topk == 0) return launch_general_quant_as<T, G, 8, 13, WIDE>(a, stream);
        if (a.stochastic) return launch_general_quant_as<T, G, 8, 12, WIDE>(a, stream);
        return launch_general_quant_as<T, G, 8, 6, WIDE>(a, stream);   // round to nearest, outliers or none
    }
    if (fixed == 6) return launch_general_quant_as<T, G, 4, 6, WIDE>(a, stream);
    if (fixed == 2) return launch_general_quant_as<T, G, 4, 2, WIDE>(a, stream);
    if (a.stochastic && a.topk == 0 && a.kind == 0) return launch_general_quant_as<T, G, 4, 13, WIDE>(a, stream);
    if (a.stochastic && a.topk == 0) return launch_general_quant_as<T, G, 4, 9, WIDE>(a, stream);
    if (fixed == 3) return launch_general_quant_as<T, G, 4, 3, CELLS, CELL_TILES>(a, stream);
    return launch_general_quant_as<T, G, 4, 0, WIDE>(a, stream);
}

template <typename T> hipError_t launch_general_quant_t(int g, int bit, const WireGeneralQuantArgs &a, hipStream_t s) {
    switch (g) {
        case 64: return launch_general_quant_g<T, 64>(bit, a, s);
        case 32: return launch_general_quant_g<T, 32>(bit, a, s);
        case 16: return launch_general_quant_g<T, 16>(bit, a, s);
        default: return hipErrorNotSupported;
    }
}

template <typename T, int G>
hipError_t launch_general_decode_g(int bit, const WireGeneralDecodeArgs &a, hipStream_t stream) {
    const int64_t tile = wire<T, 8>::TILE * kWavesPerBlock;
    const int64_t blocks = (a.numel + tile - 1) / tile;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks));
    if (bit == 8) hipLaunchKernelGGL((wire_general_decode_kernel<T, G, 8>), grid, dim3(kBlock), 0, stream, a);
    else if (bit == 4) hipLaunchKernelGGL((wire_general_decode_kernel<T, G, 4>), grid, dim3(kBlock), 0, stream, a);
    else return hipErrorNotSupported;
    return hipGetLastError();
}

template <typename T> hipError_t launch_general_decode_t(int g, int bit, const WireGeneralDecodeArgs &a, hipStream_t s) {
    switch (g) {
        case 64: return launch_general_decode_g<T, 64>(bit, a, s);
        case 32: return launch_general_decode_g<T, 32>(bit, a, s);
        case 16: return launch_general_decode_g<T, 16>(bit, a, s);
        default: return hipErrorNotSupported;
    }
}

}  // namespace

hipError_t launch_wire_general_quant(int dtype, int group_size, int bit, const WireGeneralQuantArgs &args,
                                     hipStream_t stream) {
    switch (dtype) {
        case kF32: return launch_general_quant_t<float>(group_size, bit, args, stream);
        case kF16: return launch_general_quant_t<f16>(group_size, bit, args, stream);
        case kBF16: return launch_general_quant_t<bf16>(group_size, bit, args, stream);
        default: return hipErrorNotSupported;
    }
}

hipError_t launch_wire_general_decode(int dtype, int group_size, int bit, const WireGeneralDecodeArgs &args,
                                      hipStream_t stream) {
    switch (dtype) {
        case kF32: return launch_general_decode_t<float>(group_size, bit, args, stream);
        case kF16: return launch_general_decode_t<f16>(group_size, bit, args, stream);
        case kBF16: return launch_general_decode_t<bf16>(group_size, bit, args, stream);
        default: return hipErrorNotSupported;
    }
}

}  // namespace lbc
