// One grid for two independent pieces of work of a bucket stream: the (error-feedback) quantize + pack of one
// bucket into its W chunk payloads, and the fused dequant-reduce of the W payloads that arrived for another
// bucket's shard.
//
// In the reference's reduce-scatter pipeline (ccdl_comm/communication/reduce_scatter_transport.py:262-347) the
// exchange of bucket k-1 is in flight while bucket k is quantized, so "reduce what arrived for k-1" and "quantize
// k" are ready at the same time and touch disjoint memory.  Shard-sized reduces are all launch ramp (17-41 MB of
// traffic, 5-8 us of which ~2.6 us is fixed cost); sharing the quantize's grid hides that ramp behind a kernel
// that already fills the chip: a 25 MiB bf16 bucket with fp32 residual plus the W=8 reduce of a 1.6 M-element
// shard measured 27.5 us in one grid against 29.7 us as two launches.  The reduce's workgroups come last in the
// grid (27.5 us; first 28.0 us; interleaved one to two 29.1 us).
//
// Every workgroup runs exactly the code of the separate kernels (quant_pack_block.h, dequant_reduce_block.h), so
// the results are bit-identical to lbc_quant_pack_chunks followed by lbc_dequant_reduce.
#include <type_traits>

#include "dequant_reduce_block.h"
#include "quant_pack_block.h"

namespace lbc {
namespace {

// VEC elements of the bucket per lane, as the separate quantize kernel has them: 8 for a 16-bit bucket without a
// residual, 4 for everything that touches an fp32 tensor.
template <typename XT, typename RT> constexpr int quant_vec() { return (sizeof(XT) == 2 && is_void_t<RT>::value) ? 8 : 4; }

template <typename XT, typename RT, typename OT, int W, int MODE>
__global__ __launch_bounds__(kBlock) void bucket_step_kernel(const QuantArgs q, const ReduceArgs r, unsigned quant_grid_x,
                                                            unsigned quant_blocks, unsigned reduce_blocks) {
    constexpr int G = 64, VEC = quant_vec<XT, RT>();
    using DT = typename std::conditional<VEC == 8, XT, float>::type;   // the type `restored` would have; not written here
    const unsigned b = blockIdx.x;      // wavefront-uniform: no divergence between the two bodies
    if (b < quant_blocks) {
        quant::quant_pack_block<XT, RT, DT, G, VEC, MODE>(q, b % quant_grid_x, quant_grid_x, b / quant_grid_x);
    } else {
        reduce::dequant_reduce_block<OT, G, W, MODE>(r, b - quant_blocks, reduce_blocks);
    }
}

template <typename XT, typename RT, typename OT, int W>
hipError_t launch_w(int mode, const QuantArgs &q, int quant_world, const ReduceArgs &r, hipStream_t stream) {
    using QT = quant::quant_tiling<quant_vec<XT, RT>()>;
    using RTile = reduce::decode_tiling<OT, W>;
    const int64_t padded = (q.shard_numel + 63) / 64 * 64;
    const int64_t quant_grid_x = (padded + QT::BLOCK_ELEMS - 1) / QT::BLOCK_ELEMS;
    const int64_t quant_blocks = quant_grid_x * quant_world;
    const int64_t reduce_blocks = (r.numel + RTile::BLOCK_ELEMS - 1) / RTile::BLOCK_ELEMS;
    if (quant_blocks + reduce_blocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(quant_blocks + reduce_blocks));
    if (mode == kVector)
        hipLaunchKernelGGL((bucket_step_kernel<XT, RT, OT, W, kVector>), grid, dim3(kBlock), 0, stream, q, r,
                           static_cast<unsigned>(quant_grid_x), static_cast<unsigned>(quant_blocks), static_cast<unsigned>(reduce_blocks));
    else
        hipLaunchKernelGGL((bucket_step_kernel<XT, RT, OT, W, kStream>), grid, dim3(kBlock), 0, stream, q, r,
                           static_cast<unsigned>(quant_grid_x), static_cast<unsigned>(quant_blocks), static_cast<unsigned>(reduce_blocks));
    return hipGetLastError();
}

template <typename XT, typename RT, typename OT>
hipError_t launch_o(int reduce_world, int mode, const QuantArgs &q, int quant_world, const ReduceArgs &r, hipStream_t s) {
    switch (reduce_world) {
        case 2: return launch_w<XT, RT, OT, 2>(mode, q, quant_world, r, s);
        case 4: return launch_w<XT, RT, OT, 4>(mode, q, quant_world, r, s);
        case 8: return launch_w<XT, RT, OT, 8>(mode, q, quant_world, r, s);
        default: return hipErrorNotSupported;
    }
}

template <typename XT, typename RT>
hipError_t launch_r(int x_dtype, int out_dtype, int reduce_world, int mode, const QuantArgs &q, int quant_world,
                    const ReduceArgs &r, hipStream_t s) {
    if (out_dtype == kF32) return launch_o<XT, RT, float>(reduce_world, mode, q, quant_world, r, s);
    if (out_dtype == x_dtype) return launch_o<XT, RT, XT>(reduce_world, mode, q, quant_world, r, s);
    return hipErrorNotSupported;
}

template <typename XT>
hipError_t launch_x(int x_dtype, int r_dtype, int out_dtype, int reduce_world, int mode, const QuantArgs &q,
                    int quant_world, const ReduceArgs &r, hipStream_t s) {
    if (r_dtype == kNone) return launch_r<XT, void>(x_dtype, out_dtype, reduce_world, mode, q, quant_world, r, s);
    if (r_dtype == kF32) return launch_r<XT, float>(x_dtype, out_dtype, reduce_world, mode, q, quant_world, r, s);
    return hipErrorNotSupported;
}

}  // namespace

hipError_t launch_bucket_step(int x_dtype, int r_dtype, int out_dtype, int reduce_world, int mode, const QuantArgs &quant,
                              int quant_world, const ReduceArgs &reduce, hipStream_t stream) {
    if (mode != kVector && mode != kStream) return hipErrorNotSupported;
    switch (x_dtype) {
        case kF32: return launch_x<float>(x_dtype, r_dtype, out_dtype, reduce_world, mode, quant, quant_world, reduce, stream);
        case kF16: return launch_x<f16>(x_dtype, r_dtype, out_dtype, reduce_world, mode, quant, quant_world, reduce, stream);
        case kBF16: return launch_x<bf16>(x_dtype, r_dtype, out_dtype, reduce_world, mode, quant, quant_world, reduce, stream);
        default: return hipErrorNotSupported;
    }
}

}  // namespace lbc
