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
#include "step_grid.h"

namespace lbc {
namespace {

// The quantize half is the instantiation the separate kernel would run for the same call (quant_pack_vec): VEC
// elements of the bucket per lane - 8 for a call in which every tensor is 16 bits wide, 4 as soon as an fp32 tensor
// takes part (an fp32 residual, or a 16-bit bucket without a residual whose new residual is asked for: `restored` is
// rounded to fp32 there, so the new residual is an fp32 tensor) - and DT, the type `restored` is rounded to before
// the subtraction, which fixes the new residual's type.
template <typename XT, typename RT, int VEC, typename OT, int W, int MODE>
__global__ __launch_bounds__(kBlock) void bucket_step_kernel(const QuantArgs q, const ReduceArgs r, const StepSegment quant_part,
                                                            const StepSegment reduce_part) {
    constexpr int G = 64;
    static_assert(VEC == 4 || (VEC == 8 && sizeof(XT) == 2 && is_void_t<RT>::value), "no such quantize instantiation");
    using DT = typename std::conditional<VEC == 8, XT, float>::type;
    unsigned block_x, row;              // wavefront-uniform: no divergence between the two bodies
    if (step_segment_holds(quant_part, blockIdx.x, block_x, row)) {
        if (block_x < quant_part.grid_x) quant::quant_pack_block<XT, RT, DT, G, VEC, MODE>(q, block_x, quant_part.grid_x, row);
    } else if (step_segment_holds(reduce_part, blockIdx.x, block_x, row)) {
        if (block_x < reduce_part.grid_x) reduce::dequant_reduce_block<OT, G, W, MODE>(r, block_x, reduce_part.grid_x);
    }
}

template <typename XT, typename RT, int VEC, typename OT, int W>
hipError_t launch_w(int mode, const QuantArgs &q, int quant_world, const ReduceArgs &r, hipStream_t stream) {
    using QT = quant::quant_tiling<VEC>;
    using RTile = reduce::decode_tiling<OT, W>;
    const int64_t padded = (q.shard_numel + 63) / 64 * 64;
    const int64_t quant_grid_x = (padded + QT::BLOCK_ELEMS - 1) / QT::BLOCK_ELEMS;
    const int64_t reduce_blocks = (r.numel + RTile::BLOCK_ELEMS - 1) / RTile::BLOCK_ELEMS;
    if (step_segment_slots(quant_grid_x, quant_world) + step_segment_slots(reduce_blocks, 1) > 0x7FFFFFFFLL)
        return hipErrorInvalidValue;
    int64_t cursor = 0;                 // the quantize's blocks first, the reduce's behind them
    const StepSegment quant_part = step_segment_at(cursor, quant_grid_x, quant_world);
    const StepSegment reduce_part = step_segment_at(cursor, reduce_blocks, 1);
    const dim3 grid(static_cast<unsigned>(cursor));
    if (mode == kVector)
        hipLaunchKernelGGL((bucket_step_kernel<XT, RT, VEC, OT, W, kVector>), grid, dim3(kBlock), 0, stream, q, r, quant_part, reduce_part);
    else
        hipLaunchKernelGGL((bucket_step_kernel<XT, RT, VEC, OT, W, kStream>), grid, dim3(kBlock), 0, stream, q, r, quant_part, reduce_part);
    return hipGetLastError();
}

template <typename XT, typename RT, int VEC, typename OT>
hipError_t launch_o(int reduce_world, int mode, const QuantArgs &q, int quant_world, const ReduceArgs &r, hipStream_t s) {
    switch (reduce_world) {
        case 1: return launch_w<XT, RT, VEC, OT, 1>(mode, q, quant_world, r, s);
        case 2: return launch_w<XT, RT, VEC, OT, 2>(mode, q, quant_world, r, s);
        case 3: return launch_w<XT, RT, VEC, OT, 3>(mode, q, quant_world, r, s);
        case 4: return launch_w<XT, RT, VEC, OT, 4>(mode, q, quant_world, r, s);
        case 5: return launch_w<XT, RT, VEC, OT, 5>(mode, q, quant_world, r, s);
        case 6: return launch_w<XT, RT, VEC, OT, 6>(mode, q, quant_world, r, s);
        case 7: return launch_w<XT, RT, VEC, OT, 7>(mode, q, quant_world, r, s);
        case 8: return launch_w<XT, RT, VEC, OT, 8>(mode, q, quant_world, r, s);
        default: return hipErrorNotSupported;
    }
}

template <typename XT, typename RT, int VEC>
hipError_t launch_r(int x_dtype, int out_dtype, int reduce_world, int mode, const QuantArgs &q, int quant_world,
                    const ReduceArgs &r, hipStream_t s) {
    if (out_dtype == kF32) return launch_o<XT, RT, VEC, float>(reduce_world, mode, q, quant_world, r, s);
    if (out_dtype == x_dtype) return launch_o<XT, RT, VEC, XT>(reduce_world, mode, q, quant_world, r, s);
    return hipErrorNotSupported;
}

template <typename XT>
hipError_t launch_x(int x_dtype, int r_dtype, int quant_vec, int out_dtype, int reduce_world, int mode, const QuantArgs &q,
                    int quant_world, const ReduceArgs &r, hipStream_t s) {
    if (r_dtype == kF32 && quant_vec == 4) return launch_r<XT, float, 4>(x_dtype, out_dtype, reduce_world, mode, q, quant_world, r, s);
    if (r_dtype != kNone) return hipErrorNotSupported;
    if (quant_vec == 4) return launch_r<XT, void, 4>(x_dtype, out_dtype, reduce_world, mode, q, quant_world, r, s);
    if constexpr (sizeof(XT) == 2) {
        if (quant_vec == 8) return launch_r<XT, void, 8>(x_dtype, out_dtype, reduce_world, mode, q, quant_world, r, s);
    }
    return hipErrorNotSupported;
}

}  // namespace

hipError_t launch_bucket_step(int x_dtype, int r_dtype, int quant_vec, int out_dtype, int reduce_world, int mode,
                              const QuantArgs &quant, int quant_world, const ReduceArgs &reduce, hipStream_t stream) {
    if (mode != kVector && mode != kStream) return hipErrorNotSupported;
    switch (x_dtype) {
        case kF32: return launch_x<float>(x_dtype, r_dtype, quant_vec, out_dtype, reduce_world, mode, quant, quant_world, reduce, stream);
        case kF16: return launch_x<f16>(x_dtype, r_dtype, quant_vec, out_dtype, reduce_world, mode, quant, quant_world, reduce, stream);
        case kBF16: return launch_x<bf16>(x_dtype, r_dtype, quant_vec, out_dtype, reduce_world, mode, quant, quant_world, reduce, stream);
        default: return hipErrorNotSupported;
    }
}

}  // namespace lbc
