// Device side of the decode-side kernels (fused dequant-reduce, reduce + requantize, decode of shard payloads):
// what one workgroup does.  Shared by the kernels of their own and by the kernels that carry several stages of a
// bucket stream in one grid.
#pragma once

#include "device_utils.h"
#include "launch.h"

namespace lbc {
namespace reduce {


#ifndef LBC_DECODE_UNROLL
#define LBC_DECODE_UNROLL 1
#endif
// W payloads give 2*W loads per tile; with one or two payloads a second tile in
// flight per wavefront is needed to cover the memory latency.
template <typename OT, int W = 8> struct decode_tiling {
    static constexpr int VEC = sizeof(OT) == 4 ? 4 : 8;
    static constexpr int TILE = kWave * VEC;
    static constexpr int UNROLL = W <= 2 ? 2 * LBC_DECODE_UNROLL : LBC_DECODE_UNROLL;
    static constexpr int BLOCK_ELEMS = TILE * kWavesPerBlock * UNROLL;
};

// Cache policy of the code loads in streaming mode, from measurement on 100 MiB buckets: with one to
// three payloads the output dominates the traffic and cacheable code loads are ~13 % faster; from
// four payloads on the codes dominate and the non-temporal hint wins by ~9 %.
template <int W> __device__ __forceinline__ constexpr int code_load_mode(int mode) {
    return mode == kStream && W < 4 ? kVector : mode;
}
// Cache policy of the fused reduce under the streaming modes, from sweeps of every load/store policy pair at
// W = 1, 2, 4, 8 on 3.3 M, 6.6 M and 26 M fp32 elements with buffers rotating through 650 MB.  The non-temporal
// hint pays on the direction that carries most of the bytes and costs when both directions carry it:
//   reads/writes < 0.8  (W = 1, 2 for fp32)  plain code loads, non-temporal stores       (26 M, W = 1: 19.0 us; with
//                                             non-temporal loads as well 24.8 us)
//   up to 1.6           (W = 4)               non-temporal loads; stores non-temporal, or written through for
//                                             outputs beyond the L2s
//   above               (W = 8)               non-temporal loads; plain stores while the output fits the L2s
//                                             (3.3 M: 7.9 us against 8.1 written through, 8.4 non-temporal - the
//                                             write-back then overlaps the next kernel's ramp), written through
//                                             beyond (26 M: 47.3 us against 50.2 plain, 53.6 non-temporal)
// The host picks kStream or kStreamThrough by the size of the output.  The choice holds inside a pipeline as well:
// a quantize -> shard-reduce step measured 31.7 us with these stores against 32.2-32.5 us with any other pair, and
// a 613-bucket stream of (error-feedback quantize, shard reduce) 20.69 ms against 20.8-21.2 ms.
template <typename OT, int W> constexpr int read_write_class() {
    constexpr int reads16 = W * 17, writes16 = static_cast<int>(sizeof(OT)) * 16;   // bytes per element, x16
    return reads16 * 10 < writes16 * 8 ? 0 : (reads16 * 10 < writes16 * 16 ? 1 : 2);
}
template <typename OT, int W, int MODE> constexpr int code_policy() {
    return MODE >= kStream && read_write_class<OT, W>() >= 1 ? kNtBit : kCached;
}
template <typename OT, int W, int MODE> constexpr int reduce_store_policy() {
    if (MODE < kStream) return kCached;
    if (read_write_class<OT, W>() == 0) return kNtBit;
    if (MODE == kStreamThrough) return kSc1Bit;
    return read_write_class<OT, W>() == 1 ? kNtBit : kCached;
}

template <int VEC, int MODE>
__device__ __forceinline__ void load_codes(const int8_t *__restrict__ p, uint32_t (&w)[VEC / 4]) {
    if constexpr (MODE != kScalar) {
        load_vec<uint32_t, VEC / 4, MODE>(reinterpret_cast<const uint32_t *>(p), w);
    } else {
#pragma unroll
        for (int k = 0; k < VEC / 4; ++k) {
            const uint8_t *b = reinterpret_cast<const uint8_t *>(p) + 4 * k;
            w[k] = static_cast<uint32_t>(b[0]) | (static_cast<uint32_t>(b[1]) << 8) |
                   (static_cast<uint32_t>(b[2]) << 16) | (static_cast<uint32_t>(b[3]) << 24);
        }
    }
}

// ---------------------------------------------------------------------------
// fused dequant-reduce
// ---------------------------------------------------------------------------
// One workgroup's share: block `block_x` of a grid of `grid_x` workgroups.
template <typename OT, int G, int W, int MODE>
__device__ __forceinline__ void dequant_reduce_block(const ReduceArgs &a, unsigned block_x, unsigned grid_x) {
    using T = decode_tiling<OT, W>;
    constexpr int VEC = T::VEC;
    constexpr int UNROLL = T::UNROLL;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    // every XCD walks one contiguous eighth of the shard at any size: with the policies above that measured
    // 6-15 % faster than the round-robin order from 3 M to 26 M elements (W = 8), and no slower at W = 1, 2, 4
    const int64_t block_first = static_cast<int64_t>(xcd_contiguous_block<true>(block_x, grid_x, T::BLOCK_ELEMS)) * T::BLOCK_ELEMS;
    OT *__restrict__ out = static_cast<OT *>(a.out);
    const OT *prepared = static_cast<const OT *>(a.prepared);  // may alias new_r
    OT *new_r = static_cast<OT *>(a.new_residual);
    const bool mean = a.divisor != 1.0f;

    if (MODE != kScalar && block_first + T::BLOCK_ELEMS <= a.numel) {
        // ---- interior block: one descriptor per stream over the block's span, 32-bit offsets per lane ----
        constexpr int kCodes = code_policy<OT, W, MODE>();
        constexpr int kLoad = policy_of<MODE>();
        constexpr int kStore = reduce_store_policy<OT, W, MODE>();
        uint32_t words[UNROLL][W][VEC / 4];
        float scale[UNROLL][W];
        uint32_t at[UNROLL];   // element offset inside the block
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) at[u] = static_cast<uint32_t>(tile_in_block<UNROLL>(u, wave)) * T::TILE + lane * VEC;
#pragma unroll
        for (int r = 0; r < W; ++r) {
            const buffer_t codes = buffer_over(a.codes[r] + block_first, T::BLOCK_ELEMS);
            const buffer_t scales = buffer_over(a.scales[r] + block_first / G, T::BLOCK_ELEMS / G * 4);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                buffer_load<uint32_t, VEC / 4, kCodes>(codes, at[u], words[u][r]);
                float one[1];
                buffer_load<float, 1, kCached>(scales, at[u] / G * 4, one);
                scale[u][r] = one[0];
            }
        }
        const buffer_t out_b = buffer_over(out + block_first, T::BLOCK_ELEMS * sizeof(OT));
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            float acc[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = code_to_float(words[u][0][i / 4], i % 4) * scale[u][0];
            round_through_all<OT, VEC>(acc);
#pragma unroll
            for (int r = 1; r < W; ++r) {
                float t[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) t[i] = code_to_float(words[u][r][i / 4], i % 4) * scale[u][r];
                round_through_all<OT, VEC>(t);
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[i] += t[i];
                round_through_all<OT, VEC>(acc);
            }
            if (mean) divide_all<OT, VEC>(acc, a.divisor);
            OT o[VEC];
            narrow_all<OT, VEC>(acc, o);
            buffer_store<OT, VEC, kStore>(out_b, at[u] * sizeof(OT), o);
            if (new_r != nullptr) {
                OT pv[VEC], d[VEC];
                buffer_load<OT, VEC, kLoad>(buffer_over(prepared + block_first, T::BLOCK_ELEMS * sizeof(OT)), at[u] * sizeof(OT), pv);
#pragma unroll
                for (int i = 0; i < VEC; ++i) d[i] = narrow<OT>(widen(pv[i]) - acc[i]);
                buffer_store<OT, VEC, kStore>(buffer_over(new_r + block_first, T::BLOCK_ELEMS * sizeof(OT)), at[u] * sizeof(OT), d);
            }
        }
        return;
    }

    // ---- edge block: element-wise, stores guarded by numel ----------------------
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t e0 = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * T::TILE + lane * VEC;
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            if (e >= a.numel) break;
            const int64_t g = e / G;
            float acc = 0.0f;
#pragma unroll
            for (int r = 0; r < W; ++r) {
                const float t = round_through<OT>(static_cast<float>(a.codes[r][e]) * a.scales[r][g]);
                acc = r == 0 ? t : round_through<OT>(acc + t);
            }
            if (mean) acc = round_through<OT>(acc / a.divisor);
            out[e] = narrow<OT>(acc);
            if (new_r != nullptr) new_r[e] = narrow<OT>(widen(prepared[e]) - acc);
        }
    }
}

// ---------------------------------------------------------------------------
// fused dequant-reduce + requantize (reduce-scatter shard -> all-gather payload)
// ---------------------------------------------------------------------------
// The reduced shard never reaches memory: each lane folds its 4 elements over the W payloads exactly as
// dequant_reduce_kernel does for an output of type MT (every partial sum rounded to MT, true division for
// the mean), the group maximum is taken across the lanes of the group and the codes and the scale of the
// new payload are written.  Elements past numel count as zeros, as the zero padding of a separate
// quantize would.  Reads W*(g+4)/g bytes and writes (g+4)/g bytes per element.
// Elements per lane of the fused reduce + requantize: 4 (one dword of codes per payload, 16 lanes per group
// of 64) measured 3-4 % faster on a full bucket than 8 and the same on shards.
constexpr int kReduceQuantVec = 4;
constexpr int kReduceQuantBlockElems = kWave * kReduceQuantVec * kWavesPerBlock;

// One workgroup's share: block `block_x` of a grid of `grid_x` workgroups.
template <typename MT, int G, int W, int MODE>
__device__ __forceinline__ void dequant_reduce_quant_block(const ReduceQuantArgs &a, unsigned block_x, unsigned grid_x) {
    constexpr int VEC = kReduceQuantVec;
    constexpr int LPG = G / VEC;
    constexpr int TILE = kWave * VEC;
    constexpr int BLOCK_ELEMS = TILE * kWavesPerBlock;
    static_assert(LPG >= 1 && LPG <= 16, "a group must fit one DPP row");

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t padded = (a.numel + G - 1) / G * G;
    const int64_t e0 = static_cast<int64_t>(xcd_contiguous_block<true>(block_x, grid_x, BLOCK_ELEMS)) * BLOCK_ELEMS + static_cast<int64_t>(wave) * TILE + lane * VEC;
    const bool live = e0 < padded;     // whole lanes: padded and e0 are multiples of VEC
    const bool mean = a.divisor != 1.0f;

    float p[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) p[i] = 0.0f;
    if (live) {
        uint32_t words[W][VEC / 4];
        float scale[W];
        const int64_t g = e0 / G;
#pragma unroll
        for (int r = 0; r < W; ++r) {
            load_codes<VEC, code_load_mode<W>(MODE)>(a.codes[r] + e0, words[r]);
            scale[r] = a.scales[r][g];
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) p[i] = code_to_float(words[0][i / 4], i % 4) * scale[0];
        round_through_all<MT, VEC>(p);
#pragma unroll
        for (int r = 1; r < W; ++r) {
            float t[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) t[i] = code_to_float(words[r][i / 4], i % 4) * scale[r];
            round_through_all<MT, VEC>(t);
#pragma unroll
            for (int i = 0; i < VEC; ++i) p[i] += t[i];
            round_through_all<MT, VEC>(p);
        }
        if (mean) divide_all<MT, VEC>(p, a.divisor);
        if (e0 + VEC > a.numel) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) p[i] = e0 + i < a.numel ? p[i] : 0.0f;
        }
    }
    // every lane of the row takes part in the butterfly; lanes past the end contribute zeros
    const float out_scale = group_scale<VEC, LPG>(p);
    if (!live) return;
    int c[VEC];
    encode_group<VEC>(p, out_scale, c);
    uint32_t out_words[VEC / 4];
#pragma unroll
    for (int k = 0; k < VEC / 4; ++k) out_words[k] = pack4(c[4 * k], c[4 * k + 1], c[4 * k + 2], c[4 * k + 3]);
    if constexpr (MODE != kScalar) {
        store_vec<uint32_t, VEC / 4, kVector>(reinterpret_cast<uint32_t *>(a.out_codes + e0), out_words);
    } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) a.out_codes[e0 + i] = static_cast<int8_t>(c[i]);
    }
    if ((lane & (LPG - 1)) == 0) a.out_scales[e0 / G] = out_scale;
}

// ---------------------------------------------------------------------------
// decode of one payload, or of `world` shard payloads into consecutive shards
// ---------------------------------------------------------------------------
template <int OP> __device__ __forceinline__ float combine(float old, float v) {
    if constexpr (OP == 1) return old + v;
    else if constexpr (OP == 2) return old > v ? old : v;
    else if constexpr (OP == 3) return old < v ? old : v;
    else return v;
}

#ifndef LBC_DECODE1_UNROLL
#define LBC_DECODE1_UNROLL 2
#endif
template <typename OT> struct decode1_tiling {
    static constexpr int VEC = decode_tiling<OT>::VEC;
    static constexpr int TILE = kWave * VEC;
    static constexpr int UNROLL = LBC_DECODE1_UNROLL;   // a single payload has few loads per tile: keep more tiles in flight
    static constexpr int BLOCK_ELEMS = TILE * kWavesPerBlock * UNROLL;
};

// One workgroup's share: block `block_x` of `grid_x` along shard `chunk_index`.
template <typename OT, int G, int OP, int MODE>
__device__ __forceinline__ void decode_block(const DecodeArgs &a, unsigned block_x, unsigned grid_x, unsigned chunk_index) {
    using T = decode1_tiling<OT>;
    constexpr int VEC = T::VEC;
    constexpr int UNROLL = T::UNROLL;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t chunk = chunk_index;
    const int64_t chunk_start = chunk * a.shard_numel;
    int64_t valid = a.total_numel - chunk_start;
    valid = valid < 0 ? 0 : (valid > a.shard_numel ? a.shard_numel : valid);
    const int8_t *__restrict__ codes = reinterpret_cast<const int8_t *>(a.codes_base + chunk * a.payload_stride);
    const float *__restrict__ scales = reinterpret_cast<const float *>(a.scales_base + chunk * a.payload_stride);
    OT *__restrict__ out = static_cast<OT *>(a.out) + chunk_start;
    const int64_t block_first = static_cast<int64_t>(xcd_contiguous_block(block_x, grid_x, T::BLOCK_ELEMS)) * T::BLOCK_ELEMS;
    if (block_first >= valid) return;

    if (MODE != kScalar && block_first + T::BLOCK_ELEMS <= valid) {
        uint32_t words[UNROLL][VEC / 4];
        float scale[UNROLL];
        int64_t e0[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            e0[u] = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * T::TILE + lane * VEC;
            load_codes<VEC, code_load_mode<1>(MODE)>(codes + e0[u], words[u]);
            scale[u] = scales[e0[u] / G];
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            OT o[VEC];
            if constexpr (OP != 0) load_vec<OT, VEC, MODE>(out + e0[u], o);
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                float v = round_through<OT>(code_to_float(words[u][i / 4], i % 4) * scale[u]);
                if constexpr (OP != 0) v = round_through<OT>(combine<OP>(widen(o[i]), v));
                o[i] = narrow<OT>(v);
            }
            store_vec<OT, VEC, MODE>(out + e0[u], o);
        }
        return;
    }

    for (int u = 0; u < UNROLL; ++u) {
        const int64_t e0 = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * T::TILE + lane * VEC;
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            if (e >= valid) break;
            float v = round_through<OT>(static_cast<float>(codes[e]) * scales[e / G]);
            if constexpr (OP != 0) v = round_through<OT>(combine<OP>(widen(out[e]), v));
            out[e] = narrow<OT>(v);
        }
    }
}

}  // namespace reduce
}  // namespace lbc
