// Host-side launch interface between the C ABI (lbc_api.hip) and the kernel
// translation units.  The ABI validates; these only pick an instantiation.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lbc {

constexpr int kMaxPayloads = 8;

// dtype tags shared with include/lbc.h
constexpr int kF32 = 0, kF16 = 1, kBF16 = 2, kNone = -1;

struct QuantArgs {
    const void *x;
    const void *residual;    // may be null
    uint8_t *codes_base;     // chunk d: codes at codes_base + d * payload_stride
    uint8_t *scales_base;    // chunk d: scales at scales_base + d * payload_stride
    void *new_residual;      // may be null
    void *restored;          // may be null
    void *prepared;          // may be null: x + residual in its own type, for a caller that needs it later
    int64_t numel;           // valid elements in the whole tensor
    int64_t shard_numel;     // elements per chunk (== numel for a single payload)
    int64_t payload_stride;  // bytes
};

struct ReduceArgs {
    const int8_t *codes[kMaxPayloads];
    const float *scales[kMaxPayloads];
    void *out;
    const void *prepared;  // may be null
    void *new_residual;    // may be null
    int64_t numel;
    float divisor;
};

struct ReduceQuantArgs {
    const int8_t *codes[kMaxPayloads];
    const float *scales[kMaxPayloads];
    int8_t *out_codes;     // padded: ceil(numel/g)*g codes
    float *out_scales;
    int64_t numel;
    float divisor;
};

struct DecodeArgs {
    const uint8_t *codes_base;   // chunk d: codes at codes_base + d * payload_stride
    const uint8_t *scales_base;  // chunk d: scales at scales_base + d * payload_stride
    void *out;                   // chunk d lands at out + d * shard_numel elements
    int64_t shard_numel;
    int64_t total_numel;
    int64_t payload_stride;
};

struct EfArgs {
    const void *prepared;
    const void *restored;
    void *residual;
    int64_t numel;
};

struct RingStepArgs {
    const int8_t *recv_codes;   // padded: ceil(numel/g)*g codes of the payload that arrived
    const float *recv_scales;
    void *chunk;                // numel elements, updated in place
    int8_t *send_codes;         // null together with send_scales: no payload is produced
    float *send_scales;
    int64_t numel;
    float divisor;              // 1 = no division
};

// ---- payload format of the reference's CUDA extension (cuda_wire.hip) ----------
struct WireQuantArgs {
    const void *x;
    const void *residual;    // may be null; same dtype as x
    uint8_t *payloads;       // chunk d starts at payloads + d * payload_stride
    int64_t numel;           // valid elements in the whole tensor
    int64_t shard_numel;     // elements per chunk (== numel for a single payload)
    int64_t payload_stride;  // bytes
    int compact;             // scales interleaved after each group's codes
    int nan_resets;          // group maximum as the reference's general kernels take it (a NaN resets it); needs
                             // residual == null and whole groups
};

struct WireReduceArgs {
    const uint8_t *payloads[kMaxPayloads];
    void *out;
    const void *prepared;  // may be null
    void *new_residual;    // may be null
    int64_t numel;
    float inv_divisor;
    int compact;
};

struct WireDecodeArgs {
    const uint8_t *payloads;  // chunk d starts at payloads + d * payload_stride
    void *out;                // chunk d lands at out + d * shard_numel elements
    int64_t shard_numel;
    int64_t total_numel;
    int64_t payload_stride;
    int compact;
};

struct WireRingStepArgs {
    const uint8_t *received;   // payload covering numel elements
    void *chunk;               // numel elements (a multiple of the group size), updated in place
    uint8_t *send;             // null: no payload is produced
    int64_t numel;
    float inv_divisor;         // 1 = no division
    int compact;
};

// The general policies of the CUDA extension's format (code books, stochastic rounding, top-k).
struct WireGeneralQuantArgs {
    const void *x;
    uint8_t *payload;
    int64_t numel;       // a multiple of the group size
    int kind;            // 0 linear, 1 normal, 2 uniform, 3 e3m0, 4 e2m1
    int topk;            // 0, 1, 2
    int stochastic;
    int compact;
    uint64_t seed;       // Philox key
    uint64_t offset;     // Philox offset (draws skipped in every group's stream)
};

struct WireGeneralDecodeArgs {
    const uint8_t *payload;
    void *out;
    int64_t numel;
    int kind;
    int topk;
    int compact;
    int op;              // 0 none, 1 sum, 2 max, 3 min
};

// Each returns hipSuccess/last launch error, or hipErrorNotSupported when no
// instantiation exists for the type combination.
// `mode` is an lbc::AccessMode: 0 element-wise (any alignment), 1 vector, 2 vector + non-temporal.
hipError_t launch_quant_pack(int x_dtype, int r_dtype, int d_dtype, bool outputs, int group_size, int mode,
                             const QuantArgs &args, int world, hipStream_t stream);
// Elements one lane owns for that combination (decides the alignment the vector modes need).
int quant_pack_vec(int x_dtype, int r_dtype, int d_dtype, bool outputs);
hipError_t launch_dequant_reduce(int out_dtype, int group_size, int world, int mode,
                                 const ReduceArgs &args, hipStream_t stream);
// Both of the above in one grid (group size 64; residual none or fp32; `quant_vec` = quant_pack_vec() of the quantize
// call, which also fixes the new residual's type; output fp32 or the input's type; 1 to 8 payloads; vector or
// streaming mode).  hipErrorNotSupported for anything else.
hipError_t launch_bucket_step(int x_dtype, int r_dtype, int quant_vec, int out_dtype, int reduce_world, int mode,
                              const QuantArgs &quant, int quant_world, const ReduceArgs &reduce, hipStream_t stream);
// Up to three stages of a bucket stream in one grid: chunked quantize (residual none or fp32, `quant_vec` as above),
// reduce + requantize (1 to 8 payloads) and decode of `decode_world` shard payloads, all in element type `dtype`,
// group size 64, vector or streaming mode.  A null stage is absent.  hipErrorNotSupported for anything else.
hipError_t launch_pipeline_step(int dtype, int r_dtype, int quant_vec, int mode, const QuantArgs *quant, int quant_world,
                                const ReduceQuantArgs *reduce, int reduce_world, const DecodeArgs *decode, int decode_world,
                                hipStream_t stream);
// Reduce of `world` payloads in `mid_dtype` arithmetic, requantized without leaving the chip.
hipError_t launch_dequant_reduce_quant(int mid_dtype, int group_size, int world, int mode,
                                       const ReduceQuantArgs &args, hipStream_t stream);
hipError_t launch_decode(int out_dtype, int group_size, int reduce_op, int mode,
                         const DecodeArgs &args, int world, hipStream_t stream);
// chunk (op)= decode(received) [/ divisor], then quantize+pack of the updated chunk.
hipError_t launch_ring_step(int dtype, int group_size, bool accumulate, int mode, const RingStepArgs &args,
                            hipStream_t stream);
hipError_t launch_ef_update(int p_dtype, int t_dtype, int r_dtype, int mode, const EfArgs &args,
                            hipStream_t stream);

// Wire-format launches take mode 1 (plain) or 2 (non-temporal); they have no alignment demands
// beyond element alignment.
// `bit` is 8 or 4 for quantize and decode; the fused reduce exists for 8-bit codes only.
hipError_t launch_wire_quant(int dtype, int group_size, int bit, int mode, const WireQuantArgs &args, int world,
                             hipStream_t stream);
hipError_t launch_wire_reduce(int dtype, int group_size, int world, bool fused_multiply_add, int mode,
                              const WireReduceArgs &args, hipStream_t stream);
hipError_t launch_wire_decode(int dtype, int group_size, int bit, int reduce_op, int mode, const WireDecodeArgs &args,
                              int world, hipStream_t stream);

hipError_t launch_wire_ring_step(int dtype, int group_size, bool accumulate, int mode, const WireRingStepArgs &args,
                                 hipStream_t stream);

hipError_t launch_wire_general_quant(int dtype, int group_size, int bit, const WireGeneralQuantArgs &args,
                                     hipStream_t stream);
hipError_t launch_wire_general_decode(int dtype, int group_size, int bit, const WireGeneralDecodeArgs &args,
                                      hipStream_t stream);

}  // namespace lbc
