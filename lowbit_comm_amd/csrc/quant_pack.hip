// Group-wise INT8 quantize + pack for gfx950, optionally fused with the
// error-feedback compensate (x + r) and residual update (p - restored).
//
// Mapping.  One lane owns VEC consecutive elements, so a group of G elements
// sits in G/VEC adjacent lanes of one 16-lane DPP row and the group absmax is a
// DPP butterfly with no LDS.  VEC is chosen so that the widest stream of the
// call moves 16 bytes per lane per instruction: 4 when any fp32 tensor takes
// part (input, residual, restored), 8 for a pure 16-bit call.  A wavefront
// instruction then touches one contiguous run (1 KiB for the 16-byte streams);
// a 256-thread block walks UNROLL * 4 such tiles with all loads issued before
// the first use.  Codes leave as one 4-/8-byte store per lane, the scale as one
// float from the first lane of each group.
//
// Semantics follow the reference's portable codec
// (ccdl_comm/quantization/torch_fallback.py:24-36): fp32 arithmetic, IEEE
// division for absmax/127 and p/scale, round-half-even, eps clamp on the scale.
#include "quant_pack_block.h"

namespace lbc {
namespace {

using namespace quant;

template <typename XT, typename RT, typename DT, int G, int VEC, int MODE>
__global__ __launch_bounds__(kBlock) void quant_pack_kernel(const QuantArgs a) {
    quant_pack_block<XT, RT, DT, G, VEC, MODE>(a, blockIdx.x, gridDim.x, blockIdx.y);
}

template <typename XT, typename RT, typename DT, int G, int VEC>
hipError_t launch_typed(int mode, const QuantArgs &a, int world, hipStream_t stream) {
    using T = quant_tiling<VEC>;
    const int64_t groups = (a.shard_numel + G - 1) / G;
    const int64_t padded = groups * G;
    const int64_t blocks = (padded + T::BLOCK_ELEMS - 1) / T::BLOCK_ELEMS;
    if (blocks == 0 || world == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL || world > 65535) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(world));
    switch (mode) {
        case kStream: hipLaunchKernelGGL((quant_pack_kernel<XT, RT, DT, G, VEC, kStream>), grid, dim3(kBlock), 0, stream, a); break;
        case kVector: hipLaunchKernelGGL((quant_pack_kernel<XT, RT, DT, G, VEC, kVector>), grid, dim3(kBlock), 0, stream, a); break;
        default: hipLaunchKernelGGL((quant_pack_kernel<XT, RT, DT, G, VEC, kScalar>), grid, dim3(kBlock), 0, stream, a); break;
    }
    return hipGetLastError();
}

template <typename XT, typename RT, typename DT, int VEC>
hipError_t launch_group(int g, int mode, const QuantArgs &a, int world, hipStream_t s) {
    switch (g) {
        case 64: return launch_typed<XT, RT, DT, 64, VEC>(mode, a, world, s);
        case 32: return launch_typed<XT, RT, DT, 32, VEC>(mode, a, world, s);
        case 16: return launch_typed<XT, RT, DT, 16, VEC>(mode, a, world, s);
        default: return hipErrorNotSupported;
    }
}

// residual type in {none, float, XT}; restored type in {float, XT}.  Pure 16-bit
// calls take 8 elements per lane, everything touching an fp32 tensor takes 4.
template <typename XT>
hipError_t launch_x(int x_dtype, int r_dtype, int d_dtype, bool outputs, int g, int mode, const QuantArgs &a,
                    int world, hipStream_t s) {
    constexpr int WIDE = 16 / sizeof(XT);
    const bool d_is_x = d_dtype == x_dtype;
    if (!d_is_x && d_dtype != kF32) return hipErrorNotSupported;
    if (r_dtype == kNone) {
        if (!outputs || d_is_x) return launch_group<XT, void, XT, WIDE>(g, mode, a, world, s);
        return launch_group<XT, void, float, 4>(g, mode, a, world, s);
    }
    if (r_dtype == x_dtype) {
        if (d_is_x) return launch_group<XT, XT, XT, WIDE>(g, mode, a, world, s);
        return launch_group<XT, XT, float, 4>(g, mode, a, world, s);
    }
    if (r_dtype == kF32) {
        if (d_is_x) return launch_group<XT, float, XT, 4>(g, mode, a, world, s);
        return launch_group<XT, float, float, 4>(g, mode, a, world, s);
    }
    return hipErrorNotSupported;
}

}  // namespace

int quant_pack_vec(int x_dtype, int r_dtype, int d_dtype, bool outputs) {
    if (x_dtype == kF32) return 4;
    const bool d_is_x = d_dtype == x_dtype;
    if (r_dtype == kNone) return (!outputs || d_is_x) ? 8 : 4;
    if (r_dtype == x_dtype) return d_is_x ? 8 : 4;
    return 4;
}

hipError_t launch_quant_pack(int x_dtype, int r_dtype, int d_dtype, bool outputs, int group_size, int mode,
                             const QuantArgs &args, int world, hipStream_t stream) {
    switch (x_dtype) {
        case kF32: return launch_x<float>(x_dtype, r_dtype, d_dtype, outputs, group_size, mode, args, world, stream);
        case kF16: return launch_x<f16>(x_dtype, r_dtype, d_dtype, outputs, group_size, mode, args, world, stream);
        case kBF16: return launch_x<bf16>(x_dtype, r_dtype, d_dtype, outputs, group_size, mode, args, world, stream);
        default: return hipErrorNotSupported;
    }
}

}  // namespace lbc
