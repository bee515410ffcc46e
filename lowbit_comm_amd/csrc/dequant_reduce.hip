// Decode-side kernels for gfx950: fused dequant-reduce of up to 8 payloads
// (optionally with mean and error-feedback update), single/multi-chunk decode
// with a reduce op, and the standalone error-feedback update.
//
// Mapping.  One lane owns VEC consecutive output elements: 4 for fp32 output
// (one dword of codes per payload in, one 16-byte store out) and 8 for 16-bit
// output (8 bytes of codes in, 16 bytes out), so every wavefront load and store
// is one contiguous run and the output - the largest stream - leaves as 1 KiB
// per wavefront instruction.  The lanes of one group read its scale from the
// same address (a broadcast load).  The payload pointers travel by value in the
// kernel argument block; all loads of an unrolled step are issued before the
// arithmetic starts.
//
// Semantics follow the reference's portable path: decode each payload with one
// rounding (ccdl_comm/quantization/torch_fallback.py:48-53) and add them left to
// right in list order (ccdl_comm/communication/gather_reduce.py:39-45) in the
// output dtype; "mean" is a true division (divide_all: by the bit-identical
// product with the reciprocal when the divisor is a power of two).  The translation unit is compiled
// with -ffp-contract=off so that no product/sum pair is fused into an FMA.
#include "dequant_reduce_block.h"

namespace lbc {
namespace {

using namespace reduce;

// Elements per lane of the fused reduce + requantize: 4 (one dword of codes per payload, 16 lanes per group
// of 64) measured 3-4 % faster on a full bucket than 8 and the same on shards.
constexpr int kReduceQuantVec = 4;

template <typename OT, int G, int W, int MODE>
__global__ __launch_bounds__(kBlock) void dequant_reduce_kernel(const ReduceArgs a) {
    dequant_reduce_block<OT, G, W, MODE>(a, blockIdx.x, gridDim.x);
}

template <typename OT, int G, int W>
hipError_t launch_reduce_w(int mode, const ReduceArgs &a, hipStream_t stream) {
    using T = decode_tiling<OT, W>;
    const int64_t blocks = (a.numel + T::BLOCK_ELEMS - 1) / T::BLOCK_ELEMS;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    switch (mode) {
        case kStreamThrough: hipLaunchKernelGGL((dequant_reduce_kernel<OT, G, W, kStreamThrough>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream, a); break;
        case kStream: hipLaunchKernelGGL((dequant_reduce_kernel<OT, G, W, kStream>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream, a); break;
        case kVector: hipLaunchKernelGGL((dequant_reduce_kernel<OT, G, W, kVector>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream, a); break;
        default: hipLaunchKernelGGL((dequant_reduce_kernel<OT, G, W, kScalar>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream, a); break;
    }
    return hipGetLastError();
}

template <typename OT, int G>
hipError_t launch_reduce_g(int world, int mode, const ReduceArgs &a, hipStream_t s) {
    switch (world) {
        case 1: return launch_reduce_w<OT, G, 1>(mode, a, s);
        case 2: return launch_reduce_w<OT, G, 2>(mode, a, s);
        case 3: return launch_reduce_w<OT, G, 3>(mode, a, s);
        case 4: return launch_reduce_w<OT, G, 4>(mode, a, s);
        case 5: return launch_reduce_w<OT, G, 5>(mode, a, s);
        case 6: return launch_reduce_w<OT, G, 6>(mode, a, s);
        case 7: return launch_reduce_w<OT, G, 7>(mode, a, s);
        case 8: return launch_reduce_w<OT, G, 8>(mode, a, s);
        default: return hipErrorNotSupported;
    }
}

template <typename OT>
hipError_t launch_reduce_t(int g, int world, int mode, const ReduceArgs &a, hipStream_t s) {
    switch (g) {
        case 64: return launch_reduce_g<OT, 64>(world, mode, a, s);
        case 32: return launch_reduce_g<OT, 32>(world, mode, a, s);
        case 16: return launch_reduce_g<OT, 16>(world, mode, a, s);
        default: return hipErrorNotSupported;
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
template <typename MT, int G, int W, int MODE>
__global__ __launch_bounds__(kBlock) void dequant_reduce_quant_kernel(const ReduceQuantArgs a) {
    constexpr int VEC = kReduceQuantVec;
    constexpr int LPG = G / VEC;
    constexpr int TILE = kWave * VEC;
    constexpr int BLOCK_ELEMS = TILE * kWavesPerBlock;
    static_assert(LPG >= 1 && LPG <= 16, "a group must fit one DPP row");

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t padded = (a.numel + G - 1) / G * G;
    const int64_t e0 = static_cast<int64_t>(xcd_contiguous_block<true>(BLOCK_ELEMS)) * BLOCK_ELEMS + static_cast<int64_t>(wave) * TILE + lane * VEC;
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
        for (int i = 0; i < VEC; ++i) p[i] = round_through<MT>(code_to_float(words[0][i / 4], i % 4) * scale[0]);
#pragma unroll
        for (int r = 1; r < W; ++r) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                const float t = round_through<MT>(code_to_float(words[r][i / 4], i % 4) * scale[r]);
                p[i] = round_through<MT>(p[i] + t);
            }
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

template <typename MT, int G, int W>
hipError_t launch_reduce_quant_w(int mode, const ReduceQuantArgs &a, hipStream_t stream) {
    constexpr int BLOCK_ELEMS = kWave * kReduceQuantVec * kWavesPerBlock;
    const int64_t padded = (a.numel + G - 1) / G * G;
    const int64_t blocks = (padded + BLOCK_ELEMS - 1) / BLOCK_ELEMS;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks));
    switch (mode) {
        case kStream: hipLaunchKernelGGL((dequant_reduce_quant_kernel<MT, G, W, kStream>), grid, dim3(kBlock), 0, stream, a); break;
        case kVector: hipLaunchKernelGGL((dequant_reduce_quant_kernel<MT, G, W, kVector>), grid, dim3(kBlock), 0, stream, a); break;
        default: hipLaunchKernelGGL((dequant_reduce_quant_kernel<MT, G, W, kScalar>), grid, dim3(kBlock), 0, stream, a); break;
    }
    return hipGetLastError();
}

template <typename MT, int G>
hipError_t launch_reduce_quant_g(int world, int mode, const ReduceQuantArgs &a, hipStream_t s) {
    switch (world) {
        case 1: return launch_reduce_quant_w<MT, G, 1>(mode, a, s);
        case 2: return launch_reduce_quant_w<MT, G, 2>(mode, a, s);
        case 3: return launch_reduce_quant_w<MT, G, 3>(mode, a, s);
        case 4: return launch_reduce_quant_w<MT, G, 4>(mode, a, s);
        case 5: return launch_reduce_quant_w<MT, G, 5>(mode, a, s);
        case 6: return launch_reduce_quant_w<MT, G, 6>(mode, a, s);
        case 7: return launch_reduce_quant_w<MT, G, 7>(mode, a, s);
        case 8: return launch_reduce_quant_w<MT, G, 8>(mode, a, s);
        default: return hipErrorNotSupported;
    }
}

template <typename MT>
hipError_t launch_reduce_quant_t(int g, int world, int mode, const ReduceQuantArgs &a, hipStream_t s) {
    switch (g) {
        case 64: return launch_reduce_quant_g<MT, 64>(world, mode, a, s);
        case 32: return launch_reduce_quant_g<MT, 32>(world, mode, a, s);
        case 16: return launch_reduce_quant_g<MT, 16>(world, mode, a, s);
        default: return hipErrorNotSupported;
    }
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

template <typename OT, int G, int OP, int MODE>
__global__ __launch_bounds__(kBlock) void decode_kernel(const DecodeArgs a) {
    using T = decode1_tiling<OT>;
    constexpr int VEC = T::VEC;
    constexpr int UNROLL = T::UNROLL;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t chunk = blockIdx.y;
    const int64_t chunk_start = chunk * a.shard_numel;
    int64_t valid = a.total_numel - chunk_start;
    valid = valid < 0 ? 0 : (valid > a.shard_numel ? a.shard_numel : valid);
    const int8_t *__restrict__ codes = reinterpret_cast<const int8_t *>(a.codes_base + chunk * a.payload_stride);
    const float *__restrict__ scales = reinterpret_cast<const float *>(a.scales_base + chunk * a.payload_stride);
    OT *__restrict__ out = static_cast<OT *>(a.out) + chunk_start;
    const int64_t block_first = static_cast<int64_t>(xcd_contiguous_block(T::BLOCK_ELEMS)) * T::BLOCK_ELEMS;
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

template <typename OT, int G, int OP>
hipError_t launch_decode_op(int mode, const DecodeArgs &a, int world, hipStream_t stream) {
    using T = decode1_tiling<OT>;
    const int64_t blocks = (a.shard_numel + T::BLOCK_ELEMS - 1) / T::BLOCK_ELEMS;
    if (blocks == 0 || world == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL || world > 65535) return hipErrorInvalidValue;
    dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(world));
    switch (mode) {
        case kStream: hipLaunchKernelGGL((decode_kernel<OT, G, OP, kStream>), grid, dim3(kBlock), 0, stream, a); break;
        case kVector: hipLaunchKernelGGL((decode_kernel<OT, G, OP, kVector>), grid, dim3(kBlock), 0, stream, a); break;
        default: hipLaunchKernelGGL((decode_kernel<OT, G, OP, kScalar>), grid, dim3(kBlock), 0, stream, a); break;
    }
    return hipGetLastError();
}

template <typename OT, int G>
hipError_t launch_decode_g(int op, int mode, const DecodeArgs &a, int world, hipStream_t s) {
    switch (op) {
        case 0: return launch_decode_op<OT, G, 0>(mode, a, world, s);
        case 1: return launch_decode_op<OT, G, 1>(mode, a, world, s);
        case 2: return launch_decode_op<OT, G, 2>(mode, a, world, s);
        case 3: return launch_decode_op<OT, G, 3>(mode, a, world, s);
        default: return hipErrorNotSupported;
    }
}

template <typename OT>
hipError_t launch_decode_t(int g, int op, int mode, const DecodeArgs &a, int world, hipStream_t s) {
    switch (g) {
        case 64: return launch_decode_g<OT, 64>(op, mode, a, world, s);
        case 32: return launch_decode_g<OT, 32>(op, mode, a, world, s);
        case 16: return launch_decode_g<OT, 16>(op, mode, a, world, s);
        default: return hipErrorNotSupported;
    }
}

// ---------------------------------------------------------------------------
// residual = prepared - restored
// ---------------------------------------------------------------------------
template <typename PT, typename TT, typename RT, int MODE>
__global__ __launch_bounds__(kBlock) void ef_update_kernel(const EfArgs a) {
    constexpr int VEC = 4;
    constexpr int UNROLL = 4;
    constexpr int BLOCK_ELEMS = kBlock * VEC * UNROLL;
    const PT *__restrict__ prepared = static_cast<const PT *>(a.prepared);
    const TT *__restrict__ restored = static_cast<const TT *>(a.restored);
    RT *__restrict__ residual = static_cast<RT *>(a.residual);
    const int64_t block_first = static_cast<int64_t>(xcd_contiguous_block(BLOCK_ELEMS)) * BLOCK_ELEMS;
    if (MODE != kScalar && block_first + BLOCK_ELEMS <= a.numel) {
        PT pv[UNROLL][VEC];
        TT tv[UNROLL][VEC];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t e0 = block_first + (static_cast<int64_t>(u) * kBlock + threadIdx.x) * VEC;
            load_vec<PT, VEC, MODE>(prepared + e0, pv[u]);
            load_vec<TT, VEC, MODE>(restored + e0, tv[u]);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t e0 = block_first + (static_cast<int64_t>(u) * kBlock + threadIdx.x) * VEC;
            RT d[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) d[i] = narrow<RT>(widen(pv[u][i]) - widen(tv[u][i]));
            store_vec<RT, VEC, MODE>(residual + e0, d);
        }
        return;
    }
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t e0 = block_first + (static_cast<int64_t>(u) * kBlock + threadIdx.x) * VEC;
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            if (e >= a.numel) break;
            residual[e] = narrow<RT>(widen(prepared[e]) - widen(restored[e]));
        }
    }
}

template <typename PT, typename TT, typename RT>
hipError_t launch_ef(int mode, const EfArgs &a, hipStream_t stream) {
    constexpr int BLOCK_ELEMS = kBlock * 4 * 4;
    const int64_t blocks = (a.numel + BLOCK_ELEMS - 1) / BLOCK_ELEMS;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    switch (mode) {
        case kStream: hipLaunchKernelGGL((ef_update_kernel<PT, TT, RT, kStream>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream, a); break;
        case kVector: hipLaunchKernelGGL((ef_update_kernel<PT, TT, RT, kVector>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream, a); break;
        default: hipLaunchKernelGGL((ef_update_kernel<PT, TT, RT, kScalar>), dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream, a); break;
    }
    return hipGetLastError();
}

// Supported combinations: restored has prepared's type or either is float; the
// residual has their torch promotion.  Anything else is reported unsupported.
template <typename PT, typename TT, typename RT>
hipError_t launch_ef_checked(int r_dtype, int want, int mode, const EfArgs &a, hipStream_t s) {
    if (r_dtype != want) return hipErrorNotSupported;
    return launch_ef<PT, TT, RT>(mode, a, s);
}

hipError_t launch_ef_any(int p, int t, int r, int mode, const EfArgs &a, hipStream_t s) {
    if (p == kF32 && t == kF32) return launch_ef_checked<float, float, float>(r, kF32, mode, a, s);
    if (p == kF32 && t == kF16) return launch_ef_checked<float, f16, float>(r, kF32, mode, a, s);
    if (p == kF32 && t == kBF16) return launch_ef_checked<float, bf16, float>(r, kF32, mode, a, s);
    if (p == kF16 && t == kF32) return launch_ef_checked<f16, float, float>(r, kF32, mode, a, s);
    if (p == kBF16 && t == kF32) return launch_ef_checked<bf16, float, float>(r, kF32, mode, a, s);
    if (p == kF16 && t == kF16) return launch_ef_checked<f16, f16, f16>(r, kF16, mode, a, s);
    if (p == kBF16 && t == kBF16) return launch_ef_checked<bf16, bf16, bf16>(r, kBF16, mode, a, s);
    return hipErrorNotSupported;
}

}  // namespace

hipError_t launch_dequant_reduce(int out_dtype, int group_size, int world, int mode,
                                 const ReduceArgs &args, hipStream_t stream) {
    switch (out_dtype) {
        case kF32: return launch_reduce_t<float>(group_size, world, mode, args, stream);
        case kF16: return launch_reduce_t<f16>(group_size, world, mode, args, stream);
        case kBF16: return launch_reduce_t<bf16>(group_size, world, mode, args, stream);
        default: return hipErrorNotSupported;
    }
}

hipError_t launch_dequant_reduce_quant(int mid_dtype, int group_size, int world, int mode,
                                       const ReduceQuantArgs &args, hipStream_t stream) {
    switch (mid_dtype) {
        case kF32: return launch_reduce_quant_t<float>(group_size, world, mode, args, stream);
        case kF16: return launch_reduce_quant_t<f16>(group_size, world, mode, args, stream);
        case kBF16: return launch_reduce_quant_t<bf16>(group_size, world, mode, args, stream);
        default: return hipErrorNotSupported;
    }
}

hipError_t launch_decode(int out_dtype, int group_size, int reduce_op, int mode,
                         const DecodeArgs &args, int world, hipStream_t stream) {
    switch (out_dtype) {
        case kF32: return launch_decode_t<float>(group_size, reduce_op, mode, args, world, stream);
        case kF16: return launch_decode_t<f16>(group_size, reduce_op, mode, args, world, stream);
        case kBF16: return launch_decode_t<bf16>(group_size, reduce_op, mode, args, world, stream);
        default: return hipErrorNotSupported;
    }
}

hipError_t launch_ef_update(int p_dtype, int t_dtype, int r_dtype, int mode, const EfArgs &args,
                            hipStream_t stream) {
    return launch_ef_any(p_dtype, t_dtype, r_dtype, mode, args, stream);
}

}  // namespace lbc
