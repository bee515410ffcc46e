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
// fused dequant-reduce + requantize (reduce-scatter shard -> all-gather payload): dequant_reduce_quant_block
// ---------------------------------------------------------------------------
template <typename MT, int G, int W, int MODE>
__global__ __launch_bounds__(kBlock) void dequant_reduce_quant_kernel(const ReduceQuantArgs a) {
    dequant_reduce_quant_block<MT, G, W, MODE>(a, blockIdx.x, gridDim.x);
}

template <typename MT, int G, int W>
hipError_t launch_reduce_quant_w(int mode, const ReduceQuantArgs &a, hipStream_t stream) {
    constexpr int BLOCK_ELEMS = kReduceQuantBlockElems;
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
// decode of one payload, or of `world` shard payloads into consecutive shards: decode_block
// ---------------------------------------------------------------------------
template <typename OT, int G, int OP, int MODE>
__global__ __launch_bounds__(kBlock) void decode_kernel(const DecodeArgs a) {
    decode_block<OT, G, OP, MODE>(a, blockIdx.x, gridDim.x, blockIdx.y);
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
