// Device side of quantize + pack: what one workgroup does.  Shared by the quantize kernel and by the kernel that
// carries a quantize and a fused reduce in one grid.
#pragma once

#include "device_utils.h"
#include "launch.h"

#ifndef LBC_QUANT_UNROLL
#define LBC_QUANT_UNROLL 4
#endif

namespace lbc {
namespace quant {


// torch type promotion for "a (op) b" restricted to {float, f16, bf16}.
template <typename A, typename B> struct promote { using type = float; };
template <typename A> struct promote<A, A> { using type = A; };
template <typename A> struct promote<A, void> { using type = A; };

template <typename T> struct or_float { using type = T; };
template <> struct or_float<void> { using type = float; };

// Stores of the interior blocks under the streaming mode, settled at the level of a pipeline, not of this kernel
// alone.  Without error feedback the codes are the only output and carry the non-temporal hint like the loads:
// plain or written-through code stores make the kernel 3-4 % faster when it is timed alone (26 M fp32 elements:
// 21.3 us written through, 21.4 plain, 21.9 non-temporal), but the lines they leave behind are paid for by the
// kernel that follows (a quantize -> shard-reduce step: 32.0 us non-temporal, 32.6 written through, 33.0 plain;
// the four-launch reduce-scatter plan 99.1 / 101.8 / 103.3 us).  With error feedback the residual is the large
// output and keeps the hint, and the codes are written through: a 613-bucket stream of (error-feedback quantize,
// shard reduce) measured 20.17 ms that way against 20.74 ms with both non-temporal, 20.75 both written through,
// 21.57 both plain and 21.97 the other way round; the 52 M-element bucket alone 89.9 against 93.2 us.
template <bool HAS_RESIDUAL, int MODE> constexpr int quant_code_store_policy() {
    if (MODE < kStream) return kCached;
    return HAS_RESIDUAL ? kSc1Bit : kNtBit;
}

template <int VEC> struct quant_tiling {
    static constexpr int TILE = kWave * VEC;        // elements per wavefront step
    static constexpr int UNROLL = LBC_QUANT_UNROLL; // tiles in flight per wavefront
    static constexpr int BLOCK_ELEMS = TILE * kWavesPerBlock * UNROLL;
};

// XT input, RT residual (void = none), DT type `restored` is rounded to.  Optional outputs besides the payload:
// `restored` (DT), `new_residual` = p - restored (promotion of p's type and DT) and `prepared` = p itself (p's type).
// One workgroup's share: block `block_x` of `grid_x` along the chunk, destination chunk `chunk`.
template <typename XT, typename RT, typename DT, int G, int VEC, int MODE>
__device__ __forceinline__ void quant_pack_block(const QuantArgs &a, unsigned block_x, unsigned grid_x, unsigned chunk_index) {
    using T = quant_tiling<VEC>;
    using PT = typename promote<XT, RT>::type;  // type of p = x + r
    using NT = typename promote<PT, DT>::type;  // type of p - restored
    using RLoad = typename or_float<RT>::type;  // placeholder when there is no residual
    constexpr bool HAS_R = !is_void_t<RT>::value;
    constexpr int LPG = G / VEC;                // lanes per group
    constexpr int UNROLL = T::UNROLL;
    static_assert(LPG >= 1 && LPG <= 16, "a group must fit one DPP row");

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t chunk = chunk_index;
    const int64_t chunk_start = chunk * a.shard_numel;
    int64_t valid = a.numel - chunk_start;  // live elements of this chunk
    valid = valid < 0 ? 0 : (valid > a.shard_numel ? a.shard_numel : valid);
    const int64_t groups = (a.shard_numel + G - 1) / G;
    const int64_t padded = groups * G;

    const XT *__restrict__ x = static_cast<const XT *>(a.x) + chunk_start;
    const RLoad *r = HAS_R ? static_cast<const RLoad *>(a.residual) + chunk_start : nullptr;  // may alias new_r
    int8_t *__restrict__ codes = reinterpret_cast<int8_t *>(a.codes_base + chunk * a.payload_stride);
    float *__restrict__ scales = reinterpret_cast<float *>(a.scales_base + chunk * a.payload_stride);
    NT *new_r = a.new_residual ? static_cast<NT *>(a.new_residual) + chunk_start : nullptr;
    DT *__restrict__ restored = a.restored ? static_cast<DT *>(a.restored) + chunk_start : nullptr;
    PT *__restrict__ prepared = a.prepared ? static_cast<PT *>(a.prepared) + chunk_start : nullptr;

    const int64_t block_first = static_cast<int64_t>(xcd_contiguous_block(block_x, grid_x, T::BLOCK_ELEMS)) * T::BLOCK_ELEMS;
    if (block_first >= padded) return;

    if (MODE != kScalar && block_first + T::BLOCK_ELEMS <= valid) {
        // ---- interior block: every tile is full; one descriptor per stream over the block's span ----
        constexpr int kLoad = policy_of<MODE>();
        constexpr int kSideStore = policy_of<MODE>();
        constexpr int kCodeStore = quant_code_store_policy<HAS_R, MODE>();
        XT xv[UNROLL][VEC];
        RLoad rv[UNROLL][VEC];
        uint32_t at[UNROLL];   // element offset inside the block
        const buffer_t x_b = buffer_over(x + block_first, T::BLOCK_ELEMS * sizeof(XT));
        const buffer_t r_b = buffer_over(HAS_R ? r + block_first : nullptr, T::BLOCK_ELEMS * sizeof(RLoad));
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            at[u] = static_cast<uint32_t>(tile_in_block<UNROLL>(u, wave)) * T::TILE + lane * VEC;
            buffer_load<XT, VEC, kLoad>(x_b, at[u] * sizeof(XT), xv[u]);
            if constexpr (HAS_R) buffer_load<RLoad, VEC, kLoad>(r_b, at[u] * sizeof(RLoad), rv[u]);
        }
        const buffer_t codes_b = buffer_over(codes + block_first, T::BLOCK_ELEMS);
        const buffer_t scales_b = buffer_over(scales + block_first / G, T::BLOCK_ELEMS / G * 4);
        float p[UNROLL][VEC];
        uint32_t absmax[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                float v = widen(xv[u][i]);
                if constexpr (HAS_R) v = round_through<PT>(v + widen(rv[u][i]));
                p[u][i] = v;
            }
            absmax[u] = group_absmax_bits<VEC, LPG>(p[u]);
        }
        // The scale of a group and its reciprocal cost ~18 instructions, and after the butterflies every lane of a
        // group holds the maxima of all four tiles.  With four tiles and at least four lanes per group the lanes of
        // a quad split the work: lane j of the quad takes tile j, and quad broadcasts hand the four results round.
        // Same operations on the same values as one computation per tile; 43 instructions fewer per wavefront.
        constexpr bool kSplit = UNROLL == 4 && LPG >= 4;
        float scale[UNROLL], recip[UNROLL];
        if constexpr (kSplit) {
            const int j = lane & 3;
            const uint32_t low = (j & 1) ? absmax[1] : absmax[0], high = (j & 1) ? absmax[3] : absmax[2];
            const float mine = scale_from_absmax(as_f32((j & 2) ? high : low));
            const float mine_recip = 1.0f / mine;
            scale[0] = quad_broadcast<0>(mine); recip[0] = quad_broadcast<0>(mine_recip);
            scale[1] = quad_broadcast<1>(mine); recip[1] = quad_broadcast<1>(mine_recip);
            scale[2] = quad_broadcast<2>(mine); recip[2] = quad_broadcast<2>(mine_recip);
            scale[3] = quad_broadcast<3>(mine); recip[3] = quad_broadcast<3>(mine_recip);
            if ((lane & (LPG - 1)) < 4) {     // the first quad of every group writes the four scales in one store
                const uint32_t mine_at = static_cast<uint32_t>(tile_in_block<UNROLL>(j, wave)) * T::TILE + lane * VEC;
                const float one[1] = {mine};
                buffer_store<float, 1, kCached>(scales_b, mine_at / G * 4, one);
            }
        } else {
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                scale[u] = scale_from_absmax(as_f32(absmax[u]));
                recip[u] = 1.0f / scale[u];
                if ((lane & (LPG - 1)) == 0) {
                    const float one[1] = {scale[u]};
                    buffer_store<float, 1, kCached>(scales_b, at[u] / G * 4, one);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            int c[VEC];
            const bool no_codes = scale_not_finite(scale[u]);     // then every code of the group is 0
            encode_group_finite<VEC>(p[u], scale[u], recip[u], c);

            uint32_t words[VEC / 4];
#pragma unroll
            for (int k = 0; k < VEC / 4; ++k) {                   // one select per packed word, not per code
                const uint32_t word = pack4(c[4 * k], c[4 * k + 1], c[4 * k + 2], c[4 * k + 3]);
                words[k] = no_codes ? 0u : word;
            }
            buffer_store<uint32_t, VEC / 4, kCodeStore>(codes_b, at[u], words);

            if (prepared != nullptr) {
                PT prep_out[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) prep_out[i] = narrow<PT>(p[u][i]);
                buffer_store<PT, VEC, kSideStore>(buffer_over(prepared + block_first, T::BLOCK_ELEMS * sizeof(PT)), at[u] * sizeof(PT), prep_out);
            }
            if (new_r != nullptr || restored != nullptr) {
                DT rest_out[VEC];
                NT diff_out[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const float code = no_codes ? 0.0f : code_value(c[i]);
                    const float rest = round_through<DT>(code * scale[u]);
                    rest_out[i] = narrow<DT>(rest);
                    diff_out[i] = narrow<NT>(p[u][i] - rest);
                }
                if (restored != nullptr)
                    buffer_store<DT, VEC, kSideStore>(buffer_over(restored + block_first, T::BLOCK_ELEMS * sizeof(DT)), at[u] * sizeof(DT), rest_out);
                if (new_r != nullptr)
                    buffer_store<NT, VEC, kSideStore>(buffer_over(new_r + block_first, T::BLOCK_ELEMS * sizeof(NT)), at[u] * sizeof(NT), diff_out);
            }
        }
        return;
    }

    // ---- edge block: ragged tail and zero padding, element-wise and guarded ----
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t e0 = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * T::TILE + lane * VEC;
        if (e0 - lane * VEC >= padded) break;  // wavefront-uniform
        float p[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            float v = 0.0f;
            if (e < valid) {
                v = widen(x[e]);
                if constexpr (HAS_R) v = round_through<PT>(v + widen(r[e]));
            }
            p[i] = v;
        }
        // Every lane of the row takes part in the DPP butterfly, also lanes past
        // the padded end (they contribute zeros), so no lane reads a disabled one.
        const float scale = group_scale<VEC, LPG>(p);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            const int c = encode(p[i], scale);
            if (e < padded) codes[e] = static_cast<int8_t>(c);
            if (e < valid) {
                if (prepared != nullptr) prepared[e] = narrow<PT>(p[i]);
                const float rest = round_through<DT>(static_cast<float>(c) * scale);
                if (restored != nullptr) restored[e] = narrow<DT>(rest);
                if (new_r != nullptr) new_r[e] = narrow<NT>(p[i] - rest);
            }
        }
        if ((lane & (LPG - 1)) == 0 && e0 < padded) scales[e0 / G] = scale;
    }
}

}  // namespace quant
}  // namespace lbc
