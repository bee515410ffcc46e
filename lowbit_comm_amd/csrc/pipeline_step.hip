// One grid for the three compute stages a stream of buckets has in flight at the same time under the compressed
// reduce-scatter + all-gather plan (ccdl_comm/communication/reduce_scatter_transport.py:186-377 for the first leg,
// ccdl_comm/communication/topology_transport.py:866-894 for the second):
//
//   bucket k     quantize + pack of its W destination chunks (optionally with error feedback)   -> all-to-all
//   bucket k-1   reduce of the W payloads that arrived for this rank's shard + requantize       -> all-gather
//   bucket k-2   decode of the W gathered shard payloads into the bucket
//
// The three touch disjoint memory and are ready together whenever the two exchanges of the buckets before have been
// handed to the stream, so they can share a launch: the shard-sized stages are all launch ramp on this part (a 25 MiB
// bucket's reduce + requantize moves 16 MB, its decode 40 MB), and behind a quantize that already fills the chip
// that ramp is hidden.  Any stage may be absent (the first two and the last two steps of a stream).
//
// Every workgroup runs exactly the code of the stand-alone kernels (quant_pack_block.h, dequant_reduce_block.h), so
// the results are bit-identical to lbc_quant_pack_chunks, lbc_dequant_reduce_quant and lbc_dequant_chunks.
#include <type_traits>

#include "dequant_reduce_block.h"
#include "quant_pack_block.h"
#include "step_grid.h"

namespace lbc {
namespace {

// T: element type of the bucket, of the reduce's arithmetic and of the decoded output.  RT: residual of the quantize
// (void = none).  VEC: elements per lane of the quantize, as quant_pack_vec() gives it for the same call.
template <typename T, typename RT, int VEC, int W, int MODE>
__global__ __launch_bounds__(kBlock) void bucket_pipeline_step_kernel(const QuantArgs q, const ReduceQuantArgs r, const DecodeArgs d,
                                                                     const StepSegment quant_part, const StepSegment reduce_part,
                                                                     const StepSegment decode_part) {
    constexpr int G = 64;
    static_assert(VEC == 4 || (VEC == 8 && sizeof(T) == 2 && is_void_t<RT>::value), "no such quantize instantiation");
    using DT = typename std::conditional<VEC == 8, T, float>::type;
    unsigned block_x, row;              // wavefront-uniform: no divergence between the bodies
    if (step_segment_holds(quant_part, blockIdx.x, block_x, row)) {
        if (block_x < quant_part.grid_x) quant::quant_pack_block<T, RT, DT, G, VEC, MODE>(q, block_x, quant_part.grid_x, row);
    } else if (step_segment_holds(reduce_part, blockIdx.x, block_x, row)) {
        if (block_x < reduce_part.grid_x) reduce::dequant_reduce_quant_block<T, G, W, MODE>(r, block_x, reduce_part.grid_x);
    } else if (step_segment_holds(decode_part, blockIdx.x, block_x, row)) {
        if (block_x < decode_part.grid_x) reduce::decode_block<T, G, 0, MODE>(d, block_x, decode_part.grid_x, row);
    }
}

template <typename T, typename RT, int VEC, int W>
hipError_t launch_w(int mode, const QuantArgs *q, int quant_world, const ReduceQuantArgs *r, const DecodeArgs *d,
                    int decode_world, hipStream_t stream) {
    using QT = quant::quant_tiling<VEC>;
    using DTile = reduce::decode1_tiling<T>;
    constexpr int G = 64;
    const QuantArgs qa = q ? *q : QuantArgs{};
    const ReduceQuantArgs ra = r ? *r : ReduceQuantArgs{};
    const DecodeArgs da = d ? *d : DecodeArgs{};
    const int64_t quant_grid_x = q ? ((qa.shard_numel + G - 1) / G * G + QT::BLOCK_ELEMS - 1) / QT::BLOCK_ELEMS : 0;
    const int64_t reduce_grid = r ? ((ra.numel + G - 1) / G * G + reduce::kReduceQuantBlockElems - 1) / reduce::kReduceQuantBlockElems : 0;
    const int64_t decode_grid_x = d ? (da.shard_numel + DTile::BLOCK_ELEMS - 1) / DTile::BLOCK_ELEMS : 0;
    if (step_segment_slots(quant_grid_x, quant_world) + step_segment_slots(reduce_grid, 1) +
            step_segment_slots(decode_grid_x, decode_world) > 0x7FFFFFFFLL)
        return hipErrorInvalidValue;
    // Order inside the grid, measured on 25 MiB bf16 buckets with error feedback, W = 8 (three launches: 37.2 us):
    // quantize, reduce, decode 31.2 us; reduce, quantize, decode 32.6 us; quantize, decode, reduce 33.1 us; decode,
    // quantize, reduce 34.0 us; reduce, decode, quantize 35.5 us.  The write-heavy decode goes last; the same order is
    // the fastest for 25 MiB and 100 MiB fp32 buckets.
    int64_t cursor = 0;
    const StepSegment quant_part = step_segment_at(cursor, quant_grid_x, quant_world);
    const StepSegment reduce_part = step_segment_at(cursor, reduce_grid, 1);
    const StepSegment decode_part = step_segment_at(cursor, decode_grid_x, decode_world);
    if (cursor == 0) return hipSuccess;
    const dim3 grid(static_cast<unsigned>(cursor));
    if (mode == kVector)
        hipLaunchKernelGGL((bucket_pipeline_step_kernel<T, RT, VEC, W, kVector>), grid, dim3(kBlock), 0, stream, qa, ra, da,
                           quant_part, reduce_part, decode_part);
    else
        hipLaunchKernelGGL((bucket_pipeline_step_kernel<T, RT, VEC, W, kStream>), grid, dim3(kBlock), 0, stream, qa, ra, da,
                           quant_part, reduce_part, decode_part);
    return hipGetLastError();
}

template <typename T, typename RT, int VEC>
hipError_t launch_v(int reduce_world, int mode, const QuantArgs *q, int quant_world, const ReduceQuantArgs *r,
                    const DecodeArgs *d, int decode_world, hipStream_t s) {
    switch (r ? reduce_world : 8) {       // without a reduce stage any instantiation serves
        case 1: return launch_w<T, RT, VEC, 1>(mode, q, quant_world, r, d, decode_world, s);
        case 2: return launch_w<T, RT, VEC, 2>(mode, q, quant_world, r, d, decode_world, s);
        case 3: return launch_w<T, RT, VEC, 3>(mode, q, quant_world, r, d, decode_world, s);
        case 4: return launch_w<T, RT, VEC, 4>(mode, q, quant_world, r, d, decode_world, s);
        case 5: return launch_w<T, RT, VEC, 5>(mode, q, quant_world, r, d, decode_world, s);
        case 6: return launch_w<T, RT, VEC, 6>(mode, q, quant_world, r, d, decode_world, s);
        case 7: return launch_w<T, RT, VEC, 7>(mode, q, quant_world, r, d, decode_world, s);
        case 8: return launch_w<T, RT, VEC, 8>(mode, q, quant_world, r, d, decode_world, s);
        default: return hipErrorNotSupported;
    }
}

template <typename T>
hipError_t launch_t(int r_dtype, int quant_vec, int reduce_world, int mode, const QuantArgs *q, int quant_world,
                    const ReduceQuantArgs *r, const DecodeArgs *d, int decode_world, hipStream_t s) {
    if (r_dtype == kF32 && quant_vec == 4) return launch_v<T, float, 4>(reduce_world, mode, q, quant_world, r, d, decode_world, s);
    if (r_dtype != kNone) return hipErrorNotSupported;
    if (quant_vec == 4) return launch_v<T, void, 4>(reduce_world, mode, q, quant_world, r, d, decode_world, s);
    if constexpr (sizeof(T) == 2) {
        if (quant_vec == 8) return launch_v<T, void, 8>(reduce_world, mode, q, quant_world, r, d, decode_world, s);
    }
    return hipErrorNotSupported;
}

}  // namespace

hipError_t launch_pipeline_step(int dtype, int r_dtype, int quant_vec, int mode, const QuantArgs *quant, int quant_world,
                                const ReduceQuantArgs *reduce, int reduce_world, const DecodeArgs *decode, int decode_world,
                                hipStream_t stream) {
    if (mode != kVector && mode != kStream) return hipErrorNotSupported;
    switch (dtype) {
        case kF32: return launch_t<float>(r_dtype, quant_vec, reduce_world, mode, quant, quant_world, reduce, decode, decode_world, stream);
        case kF16: return launch_t<f16>(r_dtype, quant_vec, reduce_world, mode, quant, quant_world, reduce, decode, decode_world, stream);
        case kBF16: return launch_t<bf16>(r_dtype, quant_vec, reduce_world, mode, quant, quant_world, reduce, decode, decode_world, stream);
        default: return hipErrorNotSupported;
    }
}

}  // namespace lbc
