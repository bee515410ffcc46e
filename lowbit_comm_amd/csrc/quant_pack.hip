// Group-wise INT8 quantize + pack for gfx950, optionally fused with the
// error-feedback compensate (x + r) and residual update (p - restored).
//
// Mapping.  One lane owns VEC = 16/sizeof(x) consecutive elements (one 16-byte
// load), so a 64-element group sits in 16 (fp32) or 8 (16-bit) adjacent lanes
// of one DPP row and the group absmax is a 4-/3-step DPP butterfly with no LDS.
// A wavefront instruction therefore touches 1 KiB of contiguous input; a
// 256-thread block walks UNROLL * 4 such tiles, all loads issued before the
// first use.  Codes leave as one 4-/8-byte store per lane (256/512 contiguous
// bytes per wavefront), the scale as one float from the first lane of a group.
//
// Semantics follow the reference's portable codec
// (ccdl_comm/quantization/torch_fallback.py:24-36): fp32 arithmetic, IEEE
// division for absmax/127 and p/scale, round-half-even, eps clamp on the scale.
#include "device_utils.h"
#include "launch.h"

namespace lbc {
namespace {

// torch type promotion for "a (op) b" restricted to {float, f16, bf16}.
template <typename A, typename B> struct promote { using type = float; };
template <typename A> struct promote<A, A> { using type = A; };
template <typename A> struct promote<A, void> { using type = A; };

template <typename T> struct or_float { using type = T; };
template <> struct or_float<void> { using type = float; };

template <typename XT> struct quant_tiling {
    static constexpr int VEC = 16 / sizeof(XT);
    static constexpr int TILE = kWave * VEC;                  // elements per wavefront step
    static constexpr int UNROLL = sizeof(XT) == 4 ? 4 : 2;    // tiles in flight per wavefront
    static constexpr int BLOCK_ELEMS = TILE * kWavesPerBlock * UNROLL;
};

template <typename XT, typename RT, typename DT, int G>
struct QuantLane {
    static constexpr int VEC = quant_tiling<XT>::VEC;
    static constexpr int LPG = G / VEC;  // lanes per group
    using PT = typename promote<XT, RT>::type;   // type of p = x + r
    using NT = typename promote<PT, DT>::type;   // type of p - restored
    static constexpr bool HAS_R = !is_void_t<RT>::value;
    using RLoad = typename or_float<RT>::type;  // float placeholder when there is no residual

    // p <- x (+ r), as float values already rounded to PT
    __device__ static __forceinline__ void prepare(const XT (&xv)[VEC], const float (&rv)[VEC], float (&p)[VEC]) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            float v = widen(xv[i]);
            if constexpr (HAS_R) v = round_through<PT>(v + rv[i]);
            p[i] = v;
        }
    }

    __device__ static __forceinline__ float group_scale(const float (&p)[VEC]) {
        uint32_t m = 0;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            uint32_t a = as_u32(p[i]) & 0x7FFFFFFFu;
            m = a > m ? a : m;
        }
        return scale_from_absmax(as_f32(group_max_bits<LPG>(m)));
    }
};

template <typename XT, typename RT, typename DT, int G, bool ALIGNED>
__global__ __launch_bounds__(kBlock) void quant_pack_kernel(const QuantArgs a) {
    using L = QuantLane<XT, RT, DT, G>;
    using T = quant_tiling<XT>;
    using PT = typename L::PT;
    using NT = typename L::NT;
    using RLoad = typename L::RLoad;  // float placeholder when there is no residual
    constexpr int VEC = L::VEC;
    constexpr int UNROLL = T::UNROLL;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t chunk = blockIdx.y;
    const int64_t chunk_start = chunk * a.shard_numel;
    int64_t valid = a.numel - chunk_start;            // live elements of this chunk
    valid = valid < 0 ? 0 : (valid > a.shard_numel ? a.shard_numel : valid);
    const int64_t groups = (a.shard_numel + G - 1) / G;
    const int64_t padded = groups * G;

    const XT *__restrict__ x = static_cast<const XT *>(a.x) + chunk_start;
    const RLoad *r = L::HAS_R  // may alias new_r (in-place update)
        ? static_cast<const RLoad *>(a.residual) + chunk_start : nullptr;
    int8_t *__restrict__ codes = reinterpret_cast<int8_t *>(a.codes_base + chunk * a.payload_stride);
    float *__restrict__ scales = reinterpret_cast<float *>(a.scales_base + chunk * a.payload_stride);
    NT *new_r = a.new_residual ? static_cast<NT *>(a.new_residual) + chunk_start : nullptr;
    DT *__restrict__ restored = a.restored ? static_cast<DT *>(a.restored) + chunk_start : nullptr;

    const int64_t block_first = static_cast<int64_t>(blockIdx.x) * T::BLOCK_ELEMS;
    if (block_first >= padded) return;

    if (block_first + T::BLOCK_ELEMS <= valid) {
        // ---- interior block: every tile is full, vector loads and stores -----
        XT xv[UNROLL][VEC];
        RLoad rraw[UNROLL][VEC];
        int64_t e0[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            e0[u] = block_first + static_cast<int64_t>(u * kWavesPerBlock + wave) * T::TILE + lane * VEC;
            load_vec<XT, VEC, ALIGNED>(x + e0[u], xv[u]);
            if constexpr (L::HAS_R) {
                if constexpr (sizeof(RLoad) == 4 && VEC == 8) {
                    RLoad lo[4], hi[4];
                    load_vec<RLoad, 4, ALIGNED>(r + e0[u], lo);
                    load_vec<RLoad, 4, ALIGNED>(r + e0[u] + 4, hi);
#pragma unroll
                    for (int i = 0; i < 4; ++i) { rraw[u][i] = lo[i]; rraw[u][i + 4] = hi[i]; }
                } else {
                    load_vec<RLoad, VEC, ALIGNED>(r + e0[u], rraw[u]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            float rv[VEC], p[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) rv[i] = L::HAS_R ? widen(rraw[u][i]) : 0.0f;
            L::prepare(xv[u], rv, p);
            const float scale = L::group_scale(p);
            int c[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) c[i] = encode(p[i], scale);

            uint32_t words[VEC / 4];
#pragma unroll
            for (int k = 0; k < VEC / 4; ++k) words[k] = pack4(c[4 * k], c[4 * k + 1], c[4 * k + 2], c[4 * k + 3]);
            store_vec<uint32_t, VEC / 4, ALIGNED>(reinterpret_cast<uint32_t *>(codes + e0[u]), words);
            if ((lane & (L::LPG - 1)) == 0) scales[e0[u] / G] = scale;

            if (new_r != nullptr || restored != nullptr) {
                DT rest_out[VEC];
                NT diff_out[VEC];
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const float rest = round_through<DT>(static_cast<float>(c[i]) * scale);
                    rest_out[i] = narrow<DT>(rest);
                    diff_out[i] = narrow<NT>(p[i] - rest);
                }
                if (restored != nullptr) {
                    if constexpr (sizeof(DT) * VEC == 32) {
                        DT lo[VEC / 2], hi[VEC / 2];
#pragma unroll
                        for (int i = 0; i < VEC / 2; ++i) { lo[i] = rest_out[i]; hi[i] = rest_out[i + VEC / 2]; }
                        store_vec<DT, VEC / 2, ALIGNED>(restored + e0[u], lo);
                        store_vec<DT, VEC / 2, ALIGNED>(restored + e0[u] + VEC / 2, hi);
                    } else {
                        store_vec<DT, VEC, ALIGNED>(restored + e0[u], rest_out);
                    }
                }
                if (new_r != nullptr) {
                    if constexpr (sizeof(NT) * VEC == 32) {
                        NT lo[VEC / 2], hi[VEC / 2];
#pragma unroll
                        for (int i = 0; i < VEC / 2; ++i) { lo[i] = diff_out[i]; hi[i] = diff_out[i + VEC / 2]; }
                        store_vec<NT, VEC / 2, ALIGNED>(new_r + e0[u], lo);
                        store_vec<NT, VEC / 2, ALIGNED>(new_r + e0[u] + VEC / 2, hi);
                    } else {
                        store_vec<NT, VEC, ALIGNED>(new_r + e0[u], diff_out);
                    }
                }
            }
        }
        return;
    }

    // ---- edge block: ragged tail and zero padding, element-wise and guarded ----
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t e0 = block_first + static_cast<int64_t>(u * kWavesPerBlock + wave) * T::TILE + lane * VEC;
        if (e0 - lane * VEC >= padded) break;  // wavefront-uniform
        float p[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            float v = 0.0f;
            if (e < valid) {
                v = widen(x[e]);
                if constexpr (L::HAS_R) v = round_through<PT>(v + widen(r[e]));
            }
            p[i] = v;
        }
        // Every lane of the row takes part in the DPP butterfly, also lanes past
        // the padded end (they contribute zeros), so no lane reads a disabled one.
        const float scale = L::group_scale(p);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            const int c = encode(p[i], scale);
            if (e < padded) codes[e] = static_cast<int8_t>(c);
            if (e < valid) {
                const float rest = round_through<DT>(static_cast<float>(c) * scale);
                if (restored != nullptr) restored[e] = narrow<DT>(rest);
                if (new_r != nullptr) new_r[e] = narrow<NT>(p[i] - rest);
            }
        }
        if ((lane & (L::LPG - 1)) == 0 && e0 < padded) scales[e0 / G] = scale;
    }
}

template <typename XT, typename RT, typename DT, int G>
hipError_t launch_typed(bool aligned, const QuantArgs &a, int world, hipStream_t stream) {
    using T = quant_tiling<XT>;
    const int64_t groups = (a.shard_numel + G - 1) / G;
    const int64_t padded = groups * G;
    const int64_t blocks = (padded + T::BLOCK_ELEMS - 1) / T::BLOCK_ELEMS;
    if (blocks == 0 || world == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL || world > 65535) return hipErrorInvalidValue;
    dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(world));
    if (aligned)
        hipLaunchKernelGGL((quant_pack_kernel<XT, RT, DT, G, true>), grid, dim3(kBlock), 0, stream, a);
    else
        hipLaunchKernelGGL((quant_pack_kernel<XT, RT, DT, G, false>), grid, dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

template <typename XT, typename RT, typename DT>
hipError_t launch_group(int g, bool aligned, const QuantArgs &a, int world, hipStream_t s) {
    switch (g) {
        case 64: return launch_typed<XT, RT, DT, 64>(aligned, a, world, s);
        case 32: return launch_typed<XT, RT, DT, 32>(aligned, a, world, s);
        case 16: return launch_typed<XT, RT, DT, 16>(aligned, a, world, s);
        default: return hipErrorNotSupported;
    }
}

// residual type in {none, float, XT}; restored type in {float, XT}
template <typename XT>
hipError_t launch_x(int x_dtype, int r_dtype, int d_dtype, int g, bool aligned, const QuantArgs &a, int world,
                    hipStream_t s) {
    const bool d_is_x = d_dtype == x_dtype;
    if (!d_is_x && d_dtype != kF32) return hipErrorNotSupported;
    if (r_dtype == kNone) {
        return d_is_x ? launch_group<XT, void, XT>(g, aligned, a, world, s)
                      : launch_group<XT, void, float>(g, aligned, a, world, s);
    }
    if (r_dtype == x_dtype) {
        return d_is_x ? launch_group<XT, XT, XT>(g, aligned, a, world, s)
                      : launch_group<XT, XT, float>(g, aligned, a, world, s);
    }
    if (r_dtype == kF32) {
        return d_is_x ? launch_group<XT, float, XT>(g, aligned, a, world, s)
                      : launch_group<XT, float, float>(g, aligned, a, world, s);
    }
    return hipErrorNotSupported;
}

}  // namespace

hipError_t launch_quant_pack(int x_dtype, int r_dtype, int d_dtype, int group_size, bool aligned,
                             const QuantArgs &args, int world, hipStream_t stream) {
    switch (x_dtype) {
        case kF32: return launch_x<float>(x_dtype, r_dtype, d_dtype, group_size, aligned, args, world, stream);
        case kF16: return launch_x<f16>(x_dtype, r_dtype, d_dtype, group_size, aligned, args, world, stream);
        case kBF16: return launch_x<bf16>(x_dtype, r_dtype, d_dtype, group_size, aligned, args, world, stream);
        default: return hipErrorNotSupported;
    }
}

}  // namespace lbc
