/*
 * lbc.h - C ABI of the MI355X (gfx950) low-bit communication codec.
 *
 * Plain pointers and sizes only; every pointer is a DEVICE pointer on the
 * current HIP device unless stated otherwise, every launch is asynchronous on
 * the `stream` argument (a hipStream_t passed as void*; NULL = the null
 * stream), nothing here allocates, frees or synchronises, and the only state is a
 * per-thread error string: what a call does depends on its arguments alone.
 * Inputs are never written.
 *
 * Wire format ("format A", the reference's portable codec,
 * ccdl_comm/quantization/torch_fallback.py:24-36): for a flat tensor of n
 * elements and group size g, G = ceil(n/g) groups;
 *   codes  int8[G*g]   natural element order, the tail group zero padded;
 *   scales float[G]    max(absmax/127, 2^-23) per group, IEEE division.
 * A packed payload is uint8[codes || scales] (ccdl_comm/communication/
 * payload_packing.py:63-68); passing codes = base and
 * scales = base + G*g writes or reads that layout with no copy.
 *
 * Return values: LBC_OK (0) the work was enqueued (or there was nothing to
 * do); LBC_UNSUPPORTED (1) the arguments are valid but this build has no
 * kernel for them - the caller should take its own fallback, as with the
 * reference's `return false` (ccdl_comm/csrc/quantization/
 * quant_pack_kernel.cu:231-239); negative = contract violation, text in
 * lbc_last_error() - the reference raises through TORCH_CHECK there.
 */
#ifndef LBC_H
#define LBC_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LBC_ABI_VERSION 8

enum { LBC_OK = 0, LBC_UNSUPPORTED = 1, LBC_EINVAL = -1, LBC_ELAUNCH = -2 };

/* element types: ccdl_comm/csrc/pybind.cpp:148-165 (DType) */
enum { LBC_F32 = 0, LBC_F16 = 1, LBC_BF16 = 2, LBC_NONE = -1 };

/* ccdl_comm/csrc/pybind.cpp:148-165 (ReduceOP) */
enum { LBC_REDUCE_NONE = 0, LBC_REDUCE_SUM = 1, LBC_REDUCE_MAX = 2, LBC_REDUCE_MIN = 3 };
/* QuantType of the reference (ccdl_comm/csrc/quantization/enum.cuh; code books: inner.cuh:9-35). */
enum { LBC_QUANT_LINEAR = 0, LBC_QUANT_NORMAL = 1, LBC_QUANT_UNIFORM = 2, LBC_QUANT_E3M0 = 3, LBC_QUANT_E2M1 = 4 };

#define LBC_MAX_PAYLOADS 8 /* ccdl_comm/csrc/quantization/dequant_reduce_kernel.cu:73-80,251 */

int lbc_abi_version(void);

/* Text of the last negative return on the calling thread ("" if none). */
const char *lbc_last_error(void);

/*
 * Access mode, the `access` argument of every launching entry point (no counterpart in the
 * reference).  It selects cache hints only; results never depend on it.
 *   LBC_ACCESS_AUTO    the library's rule, which looks at the call's arguments and nothing else:
 *                      today the same as LBC_ACCESS_STREAM.
 *   LBC_ACCESS_CACHED  plain cached loads and stores.  For a caller that knows the operands were
 *                      produced on this GPU a moment ago and still sit in its caches (measured ~5 %
 *                      faster than streaming then, 10-25 % slower when they do not).
 *   LBC_ACCESS_STREAM  non-temporal loads (each operand is read once); stores plain, non-temporal or
 *                      written through, as measured best per kernel and output size.
 * Operands without the alignment the vector kernels need (16 bytes for tensors, the lane's code
 * width for codes) are processed element by element under every mode.  Any other value:
 * LBC_EINVAL.
 */
enum { LBC_ACCESS_AUTO = 0, LBC_ACCESS_CACHED = 1, LBC_ACCESS_STREAM = 2 };

/*
 * Quantize + pack, optionally fused with error feedback.
 * Replaces: quantize_tensor_fallback (ccdl_comm/quantization/torch_fallback.py:10-36),
 * native inplace_quantize_pack (ccdl_comm/csrc/quantization/quant_pack_kernel.cu:220-275),
 * and, with the optional outputs, the local round trip of DDPBucketProcessor.process
 * (ccdl_comm/communication/ddp.py:69-97) plus ErrorFeedbackState.compensate/update
 * (ccdl_comm/quantization/error_feedback.py:27-41).
 *
 *   p        = x                       (residual == NULL)
 *            = x + residual            (torch promotion: any fp32 operand -> fp32 sum;
 *                                       two equal 16-bit types -> sum rounded to that type)
 *   scale_g  = max(absmax_g(p)/127, 2^-23);  code = sat8(rint(p/scale_g)), NaN -> 0
 *   restored = code*scale_g rounded to restored_dtype          (written if restored != NULL)
 *   new_residual = p - restored, rounded to new_residual_dtype (written if new_residual != NULL)
 *   prepared = p                                               (written if prepared != NULL)
 *
 * `prepared` is for the caller whose residual update comes later, from the reduced result of
 * all ranks instead of the local round trip: the reference's all_gather hook keeps
 * prepared = bucket + residual for `residual = prepared - restored` after the gather
 * (ccdl_comm/communication/ddp_hook.py:196,224-241; ErrorFeedbackState.compensate,
 * ccdl_comm/quantization/error_feedback.py:27-36), which costs it a kernel of its own before the
 * quantize.  prepared_dtype must be p's type (x_dtype without a residual, else the torch promotion
 * of x_dtype and residual_dtype); prepared must not alias another tensor of the call.
 *
 * new_residual may alias residual (in-place update).  codes must hold G*g bytes
 * and scales G floats (4-byte aligned).  Supported: group_size in {16,32,64};
 * x_dtype any; residual_dtype in {LBC_NONE, LBC_F32, x_dtype}; restored_dtype in
 * {LBC_F32, x_dtype}; new_residual_dtype must equal the torch promotion of p's
 * type and restored_dtype.  Other combinations return LBC_UNSUPPORTED.
 */
int lbc_quant_pack(const void *x, int x_dtype, const void *residual, int residual_dtype,
                   int64_t numel, int group_size, int8_t *codes, float *scales,
                   void *new_residual, int new_residual_dtype, void *restored, int restored_dtype,
                   void *prepared, int prepared_dtype, int access, void *stream);

/*
 * Quantize `world` equal destination chunks of one flat bucket in a single
 * launch, optionally fused with error feedback exactly as lbc_quant_pack
 * (residual, new_residual, restored are flat tensors of `numel` elements that
 * are indexed like x).  Replaces the per-chunk loop of the compressed
 * reduce-scatter transport (ccdl_comm/communication/reduce_scatter_transport.py:
 * 252-276,499-519) over the chunk plan of ccdl_comm/cuda/transports/
 * compressed_reduce_scatter.py:72-94: shard_numel = ceil(numel/world); the
 * bucket is treated as zero padded to world*shard_numel; chunk d covers
 * [d*shard_numel, (d+1)*shard_numel) and its groups restart at its first
 * element.  Payload d is written packed at payloads + d*payload_stride:
 * int8 codes[Gs*g] then float scales[Gs], Gs = ceil(shard_numel/g).
 * payload_stride >= Gs*(g+4) and a multiple of 4.  Pass residual =
 * new_residual = restored = prepared = NULL (dtypes ignored) for a plain quantize.
 */
int lbc_quant_pack_chunks(const void *x, int x_dtype, const void *residual, int residual_dtype,
                          int64_t numel, int world, int group_size, uint8_t *payloads,
                          int64_t payload_stride, void *new_residual, int new_residual_dtype,
                          void *restored, int restored_dtype, void *prepared, int prepared_dtype,
                          int access, void *stream);

/*
 * Decode one payload: out[i] (op)= float(code[i]) * scale[i/g], rounded to out_dtype.
 * Replaces: dequantize_tensor_fallback (ccdl_comm/quantization/torch_fallback.py:39-53)
 * and native inplace_dequantize with its ReduceOP (ccdl_comm/csrc/quantization/
 * dequant_kernel_fp32.cuh:106-120).  reduce_op NONE overwrites; SUM/MAX/MIN combine
 * with the value already in out (in out_dtype arithmetic).  numel need not be a
 * multiple of group_size; exactly numel elements are written.
 */
int lbc_dequant(const int8_t *codes, const float *scales, int64_t numel, int group_size,
                void *out, int out_dtype, int reduce_op, int access, void *stream);

/*
 * Fused dequant-reduce of `world` payloads (1..8) into one tensor, in the
 * order given, optionally fused with mean and error-feedback update.
 * Replaces: CompressedAllGatherReduce.run + _sum_tensors (ccdl_comm/communication/
 * gather_reduce.py:27-45); native try_inplace_dequantize_reduce_fused,
 * inplace_dequantize_reduce_mean and
 * inplace_dequantize_reduce_mean_update_error_feedback (ccdl_comm/csrc/quantization/
 * dequant_reduce_kernel.cu:71-134,150-221,315-430).
 *
 *   t_r   = float(code_r[i]) * scale_r[i/g]   rounded to out_dtype
 *   acc   = t_0;  acc = acc + t_r             each sum rounded to out_dtype, r = 1..world-1
 *   out   = acc                                (divisor == 1)
 *         = acc / divisor                      IEEE division in out_dtype arithmetic
 *   new_residual[i] = prepared[i] - out[i]     (if prepared != NULL; prepared_dtype must
 *                                               equal out_dtype, as must new_residual's)
 *
 * codes[] / scales[] are HOST arrays of `world` device pointers (copied by value
 * into the launch).  divisor must be > 0.  world > 8 returns LBC_UNSUPPORTED.
 */
int lbc_dequant_reduce(const int8_t *const *codes, const float *const *scales, int world,
                       int64_t numel, int group_size, float divisor, void *out, int out_dtype,
                       const void *prepared, void *new_residual, int access, void *stream);

/*
 * One launch for two independent pieces of work of a bucket stream: lbc_quant_pack_chunks of one bucket
 * (arguments x ... new_residual_dtype; `restored` is not offered) and lbc_dequant_reduce of the
 * `reduce_world` payloads that arrived for another bucket's shard (arguments codes ... reduce_new_residual),
 * both with `group_size`.  In the reference's reduce-scatter pipeline the exchange of bucket k-1 is in flight
 * while bucket k is quantized (ccdl_comm/communication/reduce_scatter_transport.py:262-347), so the two are
 * ready together; a shard-sized reduce is mostly launch ramp, and sharing the quantize's grid hides it
 * (25 MiB bf16 bucket with fp32 residual + W=8 reduce of its 1.6 M-element shard: 27.5 us against 29.7 us).
 * Results are bit-identical to the two separate calls in either order.  The reduce must not read what the
 * quantize writes: nothing orders the two inside the launch.
 * One side with nothing to do (numel == 0) launches the other alone.  LBC_UNSUPPORTED - issue the two calls
 * yourself - unless: group_size 64; every operand aligned for the vector kernels and numel/world * element
 * size a multiple of 16; residual absent or fp32; out_dtype fp32 or x_dtype (reduce_world is at most
 * 8, as for lbc_dequant_reduce).  Argument errors are reported as by the two calls.
 */
int lbc_quant_pack_chunks_and_dequant_reduce(
    const void *x, int x_dtype, const void *residual, int residual_dtype, int64_t numel, int world, int group_size,
    uint8_t *payloads, int64_t payload_stride, void *new_residual, int new_residual_dtype,
    const int8_t *const *codes, const float *const *scales, int reduce_world, int64_t reduce_numel, float divisor,
    void *out, int out_dtype, const void *prepared, void *reduce_new_residual, int access, void *stream);

/*
 * Decode `world` payloads into `world` consecutive shards of one flat tensor in a
 * single launch (the all-gather leg: ccdl_comm/communication/topology_transport.py:
 * 866-894 decodes every gathered shard payload into its slot).  Payload d is
 * packed at payloads + d*payload_stride as written by lbc_quant_pack_chunks for a
 * shard of shard_numel elements; shard d lands at out + d*shard_numel; only the
 * first total_numel elements of the concatenation are written.
 */
int lbc_dequant_chunks(const uint8_t *payloads, int64_t payload_stride, int world,
                       int64_t shard_numel, int64_t total_numel, int group_size, void *out,
                       int out_dtype, int access, void *stream);

/*
 * Fused reduce + requantize for the reduce-scatter -> all-gather hand-over: the payload of
 * quantize(reduce(payloads)) without writing the reduced shard.  The reduce is the one of
 * lbc_dequant_reduce for an output of type mid_dtype (list order, every partial sum rounded to
 * mid_dtype, true division by divisor), the quantize the one of lbc_quant_pack on that result,
 * elements past numel counting as zeros.  Replaces the two steps
 * `_dequantize_reduce_payloads` + `_quantize_chunk` of the topology transport when no caller needs
 * the full-precision shard (ccdl_comm/communication/topology_transport.py:866-894 gathers and decodes
 * only the requantized payloads).  out_codes holds ceil(numel/g)*g codes, out_scales ceil(numel/g)
 * floats; neither may alias an input.  world > 8: LBC_UNSUPPORTED.
 */
int lbc_dequant_reduce_quant(const int8_t *const *codes, const float *const *scales, int world,
                             int64_t numel, int group_size, float divisor, int mid_dtype,
                             int8_t *out_codes, float *out_scales, int access, void *stream);

/*
 * One launch for the three compute stages that a stream of buckets has in flight together under the
 * compressed reduce-scatter + all-gather plan: the chunked quantize of bucket k (its all-to-all follows),
 * the reduce + requantize of the payloads that arrived for bucket k-1's shard (its all-gather follows) and
 * the decode of the gathered shard payloads of bucket k-2.  In the reference these are the compute steps
 * between the collectives of ccdl_comm/communication/reduce_scatter_transport.py:252-347 (quantize the
 * chunks, reduce what arrived) and ccdl_comm/communication/topology_transport.py:866-894 (requantize,
 * gather, decode every shard), one kernel each and one bucket at a time; consecutive DDP buckets are
 * independent, so stage s of bucket k-s is ready when the exchanges of the earlier buckets have been
 * handed to the stream, and the shard-sized stages, which are mostly launch ramp on their own, ride in
 * the grid of the quantize.
 *
 * Each stage structure carries the arguments of the call it stands for - lbc_quant_pack_chunks (without
 * `restored` and `prepared`), lbc_dequant_reduce_quant, lbc_dequant_chunks - with the same meaning and
 * the same validation; a NULL stage is absent, and a stage with nothing to do (numel == 0) counts as
 * absent.  Results are bit-identical to those calls in any order.  Nothing orders the stages inside the
 * launch: no stage may read or write what another writes (LBC_EINVAL otherwise; decoding bucket k-2 in
 * place is fine, its quantize ran two launches earlier).
 *
 * With one stage present its own kernel runs.  With two or three: LBC_UNSUPPORTED - issue the calls
 * yourself - unless group_size is 64, every operand is aligned for the vector kernels (16 bytes for
 * tensors and shard boundaries, 4 for payload rows; 8 for 16-bit output), the residual is absent or
 * fp32, and x_dtype, mid_dtype and out_dtype are one type (the reduce has at most 8 payloads, as always).
 */
typedef struct lbc_quant_chunks_stage {
    const void *x;
    const void *residual;       /* may be NULL */
    uint8_t *payloads;
    void *new_residual;         /* may be NULL; may alias residual */
    int64_t numel;
    int64_t payload_stride;
    int x_dtype, residual_dtype, new_residual_dtype, world;
} lbc_quant_chunks_stage;

typedef struct lbc_reduce_quant_stage {
    const int8_t *const *codes;  /* HOST arrays of `world` device pointers */
    const float *const *scales;
    int8_t *out_codes;
    float *out_scales;
    int64_t numel;
    float divisor;
    int world, mid_dtype;
} lbc_reduce_quant_stage;

typedef struct lbc_dequant_chunks_stage {
    const uint8_t *payloads;
    void *out;
    int64_t payload_stride;
    int64_t shard_numel;
    int64_t total_numel;
    int world, out_dtype;
} lbc_dequant_chunks_stage;

int lbc_bucket_pipeline_step(const lbc_quant_chunks_stage *quant, const lbc_reduce_quant_stage *reduce,
                             const lbc_dequant_chunks_stage *decode, int group_size, int access,
                             void *stream);

/*
 * One compute step of the quantized ring all-reduce on one chunk of the bucket, in place:
 *   chunk[i] = decode(received)[i]                      reduce_op LBC_REDUCE_NONE
 *   chunk[i] = chunk[i] + decode(received)[i]           reduce_op LBC_REDUCE_SUM (in `dtype` arithmetic)
 *   chunk[i] = chunk[i] / divisor                       when divisor != 1 (true division)
 * and, when send_codes and send_scales are given, quantize+pack of the updated chunk exactly as
 * lbc_quant_pack would, without reading it back from memory.  Replaces, in one launch,
 * TorchPipelinedRingRuntime.fused_reduce / apply_broadcast (ccdl_comm/cuda/transports/
 * torch_topology.py:262-316: dequantize with reduce_op sum / none, div_ by the world size at the
 * last reduce step) followed by the quant_pack of the same chunk that the ring schedule issues
 * next (ccdl_comm/cuda/transports/pipelined_ring.py:221-225,250-254; the chunk a step receives
 * into is the chunk the next step sends, :304-311,325-330).  Results are bit-identical to
 * lbc_dequant + division + lbc_quant_pack.  recv_codes holds ceil(numel/g)*g codes, recv_scales
 * ceil(numel/g) floats; the send buffers have the same sizes and may not alias the received
 * ones.  Other reduce ops: LBC_UNSUPPORTED.
 */
int lbc_ring_step(const int8_t *recv_codes, const float *recv_scales, void *chunk, int dtype,
                  int64_t numel, int group_size, int reduce_op, float divisor, int8_t *send_codes,
                  float *send_scales, int access, void *stream);

/*
 * residual = prepared - restored, element-wise, subtraction in fp32, rounded to
 * residual_dtype.  Supported: restored_dtype equal to prepared_dtype or either of
 * them LBC_F32, and residual_dtype their torch promotion; else LBC_UNSUPPORTED.  Replaces native inplace_error_feedback_update (ccdl_comm/csrc/
 * quantization/dequant_reduce_kernel.cu:136-148,223-233,266-313) and
 * ErrorFeedbackState.update (ccdl_comm/quantization/error_feedback.py:38-41).
 */
int lbc_ef_update(const void *prepared, int prepared_dtype, const void *restored, int restored_dtype,
                  void *residual, int residual_dtype, int64_t numel, int access, void *stream);

/* ------------------------------------------------------------------------------------------
 * Payload format of the reference's CUDA extension ("format B", the bytes ccdl_cuda_ops
 * produces and consumes), for fleets that mix ranks running that extension with gfx950 ranks.
 * `dtype` is the element type of the tensor AND of the stored scales; G = ceil(n/g) groups:
 *   scale  = max |p| over the group, stored as `dtype` (NaNs are skipped);
 *   code   = rint(p * (127 / max(float(scale), 1e-6f))), NaN -> 0
 *            (ccdl_comm/csrc/quantization/quant_pack_kernel.cu:86-103,111-143);
 *   bytes  = codes with the byte order reversed inside every sizeof(dtype)-byte word;
 *   compact != 0: per group [g code bytes][scale]  (quant_pack_kernel.cu:104-106,160-162)
 *   compact == 0: all code bytes, then all scales  (quant_kernel_fp32.cuh:266-303);
 *   decode = float(code) * (float(scale) / 127), rounded to `dtype`
 *            (dequant_reduce_kernel.cu:38-69, dequant_kernel_fp32.cuh:81-104).
 * `bit` = 4 selects 4-bit codes: multiplier 7 / max(scale, 1e-6), two's-complement nibbles packed
 * 2*sizeof(dtype) to a word with the first code in the most significant nibble, decode by scale / 7
 * (quant_pack_kernel.cu:103,120-130,145-158; ccdl_comm/csrc/quantization/inner.cuh:36-40,67-72).
 * A payload holds G * (g*bit/8 + sizeof(dtype)) bytes and must be aligned to sizeof(dtype).
 * No golden bytes of an NVIDIA build exist in the reference, so byte equality with such a
 * build is argued from the source, not measured.
 */

/* Bytes of one payload (quant_pack_kernel.cu:247-249); -1 for invalid arguments. */
int64_t lbc_wire_payload_nbytes(int64_t numel, int group_size, int dtype, int bit);

/*
 * Quantize x (+ residual, added in fp32 and rounded to dtype first) into one payload.
 * Replaces native inplace_quantize_pack and inplace_quantize for linear 8- and 4-bit codes
 * (quant_pack_kernel.cu:220-275, ccdl_comm/csrc/pybind.cpp:36-63).  Ragged numel is zero padded.
 * NaN elements: the reference sends a call without a residual whose numel is a multiple of
 * group_size to its general kernels, whose running group maximum `(m > a) ? m : a` a NaN resets
 * (utils.cuh:11, quant_kernel_fp32.cuh:93-97), and every other call to its pack kernel, whose
 * fmaxf skips NaNs (quant_pack_kernel.cu:259-262,94-99); this entry point makes the same choice
 * per call (per chunk in the chunked form).
 */
int lbc_wire_quant_pack(const void *x, const void *residual, int dtype, int64_t numel, int group_size,
                        int bit, int compact, uint8_t *payload, int access, void *stream);

/* As lbc_quant_pack_chunks, in this format: chunk d of ceil(numel/world) elements becomes the
 * payload at payloads + d*payload_stride (ccdl_comm/cuda/transports/compressed_reduce_scatter.py:72-94). */
int lbc_wire_quant_pack_chunks(const void *x, const void *residual, int dtype, int64_t numel, int world,
                               int group_size, int bit, int compact, uint8_t *payloads,
                               int64_t payload_stride, int access, void *stream);

/*
 * Decode one payload into out (reduce_op NONE) or combine it with the values already in out:
 * SUM adds in `dtype` with one rounding, MAX/MIN keep `(old > new) ? old : new` resp. its
 * opposite.  Replaces native inplace_dequantize (dequant_kernel_fp32.cuh:106-120,
 * dequant_kernel.cuh:46-60, pybind.cpp:64-90).
 */
int lbc_wire_dequant(const uint8_t *payload, int64_t numel, int group_size, int bit, int compact, void *out,
                     int dtype, int reduce_op, int access, void *stream);

/* As lbc_dequant_chunks, in this format (ccdl_comm/communication/topology_transport.py:866-894). */
int lbc_wire_dequant_chunks(const uint8_t *payloads, int64_t payload_stride, int world, int64_t shard_numel,
                            int64_t total_numel, int group_size, int bit, int compact, void *out, int dtype,
                            int reduce_op, int access, void *stream);

/*
 * out = dtype(sum_r float(code_r) * (scale_r / 127) * inv_divisor), payloads added in list order in
 * fp32 starting from 0; with prepared/new_residual: new_residual = dtype(float(prepared) - the
 * unrounded fp32 value).  Replaces native try_inplace_dequantize_reduce_fused and
 * inplace_dequantize_reduce_mean_update_error_feedback (dequant_reduce_kernel.cu:71-134,150-221,
 * 315-430), which support 8-bit codes, group_size 64 and world <= 8 only; so does this.
 * fused_multiply_add != 0 accumulates with fma(code, step, sum), which is what nvcc's default
 * contraction makes of the reference's `sum += code * step`; 0 rounds the product first.
 */
int lbc_wire_dequant_reduce(const uint8_t *const *payloads, int world, int64_t numel, int group_size,
                            int compact, float inv_divisor, int fused_multiply_add, void *out, int dtype,
                            const void *prepared, void *new_residual, int access, void *stream);

/*
 * One hop of the quantized ring or tree in this format, in place on a chunk of whole groups:
 *   chunk[i] = decode(received)[i]                   reduce_op LBC_REDUCE_NONE
 *   chunk[i] = chunk[i] + decode(received)[i]        reduce_op LBC_REDUCE_SUM (one rounding to `dtype`)
 *   chunk[i] = chunk[i] * (1 / divisor)              when divisor != 1: what `tensor.div_(W)` computes on a
 *                                                    device tensor (float reciprocal, rounded to `dtype`)
 * and, when `send` is given, the payload lbc_wire_quant_pack would write for the updated chunk (linear 8-bit
 * codes), in the same launch.  Replaces TorchPipelinedRingRuntime / TorchTreeRuntime .fused_reduce and
 * .apply_broadcast with the extension loaded (ccdl_comm/cuda/transports/torch_topology.py:262-316,367-415:
 * inplace_dequantize with SUM / NONE, div_) plus the quant_pack of the same chunk that follows
 * (pipelined_ring.py:221-225,250-254).  numel must be a multiple of group_size, as the reference's in-place
 * decode demands (torch_topology.py:205-214); `send` must not alias `received`.  Other reduce ops:
 * LBC_UNSUPPORTED.
 */
int lbc_wire_ring_step(const uint8_t *received, void *chunk, int dtype, int64_t numel, int group_size,
                       int compact, int reduce_op, float divisor, uint8_t *send, int access, void *stream);

/*
 * The remaining policies of the CUDA extension's format: non-linear 4-bit code books
 * (quant_type != LINEAR needs bit == 4), stochastic rounding and the top-k side channel
 * (topk 0, 1, 2), in any combination.  numel must be a multiple of group_size, as in the reference
 * (gen_code_quant.py:164).  A group's bytes are [codes][scale][indices][top1][top2] in words of the
 * tensor's item size, the metadata behind each group (compact) or behind all codes; the group
 * maximum is the reference's running `(m > a) ? m : a`, which a NaN resets.
 */
int64_t lbc_wire_general_payload_nbytes(int64_t numel, int group_size, int dtype, int bit, int topk);

/*
 * Replaces native quantize / inplace_quantize (gen_code_quant.py:162-277 dispatching to
 * quant_kernel_fp32.cuh:211-455 and quant_kernel.cuh:155-399).  With stochastic != 0, seed and offset are
 * the Philox key and offset the reference takes from torch's CUDA generator
 * (gen_code_quant.py:27-36: philox_engine_inputs(numel)); group s draws from subsequence s.
 * A policy with nothing general about it (linear codes, topk 0, no stochastic rounding) is handed to the
 * kernel of lbc_wire_quant_pack, which writes the same bytes at the memory-bound rate.
 */
int lbc_wire_quant_general(const void *x, int dtype, int64_t numel, int group_size, int bit, int quant_type,
                           int topk, int stochastic, uint64_t seed, uint64_t offset, int compact,
                           uint8_t *payload, void *stream);

/* Replaces native dequantize / inplace_dequantize for those policies (dequant_kernel_fp32.cuh:122-353,
 * dequant_kernel.cuh:62-291); reduce_op as in lbc_wire_dequant.  Linear codes without an outlier channel
 * (however they were rounded) are decoded by the kernel of lbc_wire_dequant. */
int lbc_wire_dequant_general(const uint8_t *payload, int64_t numel, int group_size, int bit, int quant_type,
                             int topk, int compact, void *out, int dtype, int reduce_op, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LBC_H */
