// C ABI of the codec library (declared in include/lbc.h): argument validation,
// alignment probing and dispatch.  No allocation, no synchronisation, no state
// besides a per-thread error string: what a call does is a function of its arguments.
#include "../../include/lbc.h"

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

#include "launch.h"

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

bool valid_dtype(int d) { return d == LBC_F32 || d == LBC_F16 || d == LBC_BF16; }
int dtype_size(int d) { return d == LBC_F32 ? 4 : 2; }
bool valid_group(int g) { return g == 16 || g == 32 || g == 64; }

bool aligned_to(const void *p, uintptr_t bytes) { return (reinterpret_cast<uintptr_t>(p) & (bytes - 1)) == 0; }

// torch promotion of two of {f32, f16, bf16}
int promote(int a, int b) { return a == b ? a : LBC_F32; }

// Access mode of a call (LBC_ACCESS_*): a function of the arguments only, no process state.  Operands that lack
// the alignment of the vector paths take the element-wise kernels whatever the caller asked for.
bool valid_access(int access) { return access >= LBC_ACCESS_AUTO && access <= LBC_ACCESS_STREAM; }

int pick_mode(bool aligned, int access) {
    if (!aligned) return 0;
    return access == LBC_ACCESS_CACHED ? 1 : 2;
}

// The fused reduce writes through once a streaming call's output is well beyond the 32 MiB of L2; smaller outputs
// stay in plain cached stores, whose write-back then overlaps with whatever runs next.
int pick_mode(bool aligned, int access, int64_t written_bytes) {
    const int mode = pick_mode(aligned, access);
    return mode == 2 && written_bytes >= (int64_t{24} << 20) ? 3 : mode;
}

int finish(hipError_t err, const char *what) {
    if (err == hipSuccess) return LBC_OK;
    if (err == hipErrorNotSupported) return LBC_UNSUPPORTED;
    return fail(LBC_ELAUNCH, "%s: %s", what, hipGetErrorString(err));
}

}  // namespace

namespace {

// A validated call, ready to launch.  status != LBC_OK: return it (nothing to launch); `empty`: LBC_OK with no work.
struct QuantCall {
    int status = LBC_OK;
    bool empty = false;
    lbc::QuantArgs args{};
    int x_dtype = LBC_F32, r_dtype = LBC_NONE, d_dtype = LBC_F32, world = 1, group_size = 64;
    bool outputs = false, aligned = false;
};

struct ReduceCall {
    int status = LBC_OK;
    bool empty = false;
    lbc::ReduceArgs args{};
    int out_dtype = LBC_F32, world = 0, group_size = 64;
    bool aligned = false;
};

struct ReduceQuantCall {
    int status = LBC_OK;
    bool empty = false;
    lbc::ReduceQuantArgs args{};
    int mid_dtype = LBC_F32, world = 0;
    bool aligned = false;
};

struct DecodeCall {
    int status = LBC_OK;
    bool empty = false;
    lbc::DecodeArgs args{};
    int out_dtype = LBC_F32, world = 0;
    bool aligned = false;
};

QuantCall refuse_quant(int status) { QuantCall c; c.status = status; return c; }
ReduceQuantCall refuse_reduce_quant(int status) { ReduceQuantCall c; c.status = status; return c; }
DecodeCall refuse_decode(int status) { DecodeCall c; c.status = status; return c; }
ReduceCall refuse_reduce(int status) { ReduceCall c; c.status = status; return c; }

// Shared body of lbc_quant_pack (world == 1, separate codes/scales pointers) and
// lbc_quant_pack_chunks (world >= 1, packed rows): dtype rules and alignment.
QuantCall quant_pack_common(const void *x, int x_dtype, const void *residual, int residual_dtype,
                            int64_t numel, int world, int group_size, uint8_t *codes_base, uint8_t *scales_base,
                            int64_t payload_stride, int64_t shard_numel, void *new_residual, int new_residual_dtype,
                            void *restored, int restored_dtype, void *prepared, int prepared_dtype) {
    const int r_dtype = residual ? residual_dtype : LBC_NONE;
    const int p_dtype = residual ? promote(x_dtype, r_dtype) : x_dtype;
    if (prepared != nullptr && prepared_dtype != p_dtype)
        return refuse_quant(fail(LBC_EINVAL, "prepared must have the promoted dtype of input and residual"));
    if (prepared != nullptr && (prepared == x || prepared == residual || prepared == new_residual || prepared == restored))
        return refuse_quant(fail(LBC_EINVAL, "prepared must not alias another tensor of the call"));
    if (prepared != nullptr && !aligned_to(prepared, dtype_size(p_dtype)))
        return refuse_quant(fail(LBC_EINVAL, "prepared is not aligned to its element size"));
    const bool wants_outputs = new_residual != nullptr || restored != nullptr;
    int d_dtype = LBC_F32;
    if (wants_outputs) {
        if (!valid_dtype(restored_dtype)) return refuse_quant(fail(LBC_EINVAL, "unsupported restored dtype %d", restored_dtype));
        d_dtype = restored_dtype;
        if (new_residual != nullptr) {
            if (!valid_dtype(new_residual_dtype))
                return refuse_quant(fail(LBC_EINVAL, "unsupported new-residual dtype %d", new_residual_dtype));
            if (new_residual_dtype != promote(p_dtype, d_dtype))
                return refuse_quant(fail(LBC_EINVAL, "new residual must have the promoted dtype of (input+residual) and restored"));
        }
    }
    if (r_dtype != LBC_NONE && r_dtype != LBC_F32 && r_dtype != x_dtype) return refuse_quant(LBC_UNSUPPORTED);
    if (d_dtype != LBC_F32 && d_dtype != x_dtype) return refuse_quant(LBC_UNSUPPORTED);

    const int vec = lbc::quant_pack_vec(x_dtype, r_dtype, d_dtype, wants_outputs);
    bool aligned = aligned_to(x, 16) && aligned_to(codes_base, vec) && payload_stride % vec == 0;
    auto side = [&](const void *p, int dtype) {
        if (p == nullptr) return;
        aligned = aligned && aligned_to(p, 16) && (world == 1 || (shard_numel * dtype_size(dtype)) % 16 == 0);
    };
    if (world > 1) aligned = aligned && (shard_numel * dtype_size(x_dtype)) % 16 == 0;
    side(residual, r_dtype);
    side(new_residual, new_residual_dtype);
    side(restored, d_dtype);
    side(prepared, p_dtype);

    QuantCall c;
    c.args.x = x;
    c.args.residual = residual;
    c.args.codes_base = codes_base;
    c.args.scales_base = scales_base;
    c.args.new_residual = new_residual;
    c.args.restored = restored;
    c.args.prepared = prepared;
    c.args.numel = numel;
    c.args.shard_numel = shard_numel;
    c.args.payload_stride = payload_stride;
    c.x_dtype = x_dtype;
    c.r_dtype = r_dtype;
    c.d_dtype = d_dtype;
    c.world = world;
    c.group_size = group_size;
    c.outputs = wants_outputs;
    c.aligned = aligned;
    return c;
}

int launch_quant(const QuantCall &c, const char *what, int access, void *stream) {
    if (c.status != LBC_OK || c.empty) return c.status;
    return finish(lbc::launch_quant_pack(c.x_dtype, c.r_dtype, c.d_dtype, c.outputs, c.group_size,
                                         pick_mode(c.aligned, access), c.args, c.world, static_cast<hipStream_t>(stream)),
                  what);
}

// Validation of lbc_quant_pack_chunks, shared with the entry point that carries a reduce in the same launch.
QuantCall prepare_quant_chunks(const void *x, int x_dtype, const void *residual, int residual_dtype, int64_t numel,
                               int world, int group_size, uint8_t *payloads, int64_t payload_stride, void *new_residual,
                               int new_residual_dtype, void *restored, int restored_dtype, void *prepared,
                               int prepared_dtype) {
    if (numel < 0) return refuse_quant(fail(LBC_EINVAL, "numel must be >= 0"));
    if (world <= 0) return refuse_quant(fail(LBC_EINVAL, "world must be > 0"));
    if (!valid_dtype(x_dtype)) return refuse_quant(fail(LBC_EINVAL, "unsupported input dtype %d", x_dtype));
    if (residual != nullptr && !valid_dtype(residual_dtype))
        return refuse_quant(fail(LBC_EINVAL, "unsupported residual dtype %d", residual_dtype));
    if (!valid_group(group_size)) return refuse_quant(LBC_UNSUPPORTED);
    if (world > 65535) return refuse_quant(LBC_UNSUPPORTED);
    const int64_t shard = (numel + world - 1) / world;
    if (shard == 0) {
        QuantCall c;
        c.empty = true;
        return c;
    }
    const int64_t groups = (shard + group_size - 1) / group_size;
    const int64_t payload_bytes = groups * (group_size + 4);
    if (x == nullptr || payloads == nullptr) return refuse_quant(fail(LBC_EINVAL, "input and payloads must not be null"));
    if (payload_stride < payload_bytes || (payload_stride & 3) != 0)
        return refuse_quant(fail(LBC_EINVAL, "payload_stride must be a multiple of 4 and >= %lld", (long long)payload_bytes));
    if (!aligned_to(payloads, 4)) return refuse_quant(fail(LBC_EINVAL, "payloads must be 4-byte aligned"));
    if (!aligned_to(x, dtype_size(x_dtype))) return refuse_quant(fail(LBC_EINVAL, "input is not aligned to its element size"));
    return quant_pack_common(x, x_dtype, residual, residual_dtype, numel, world, group_size, payloads,
                             payloads + groups * group_size, payload_stride, shard, new_residual, new_residual_dtype,
                             restored, restored_dtype, prepared, prepared_dtype);
}

// Validation of lbc_dequant_reduce, shared in the same way.
ReduceCall prepare_reduce(const int8_t *const *codes, const float *const *scales, int world, int64_t numel,
                          int group_size, float divisor, void *out, int out_dtype, const void *prepared,
                          void *new_residual) {
    if (world <= 0) return refuse_reduce(fail(LBC_EINVAL, "inputs must not be empty"));
    if (numel < 0) return refuse_reduce(fail(LBC_EINVAL, "numel must be >= 0"));
    if (!(divisor > 0.0f)) return refuse_reduce(fail(LBC_EINVAL, "divisor must be > 0"));
    if (!valid_dtype(out_dtype)) return refuse_reduce(fail(LBC_EINVAL, "unsupported output dtype %d", out_dtype));
    if ((prepared == nullptr) != (new_residual == nullptr))
        return refuse_reduce(fail(LBC_EINVAL, "prepared and new_residual must be given together"));
    if (world > LBC_MAX_PAYLOADS || !valid_group(group_size)) return refuse_reduce(LBC_UNSUPPORTED);
    ReduceCall c;
    if (numel == 0) {
        c.empty = true;
        return c;
    }
    if (codes == nullptr || scales == nullptr || out == nullptr)
        return refuse_reduce(fail(LBC_EINVAL, "codes, scales and out must not be null"));
    const int vec = out_dtype == LBC_F32 ? 4 : 8;
    bool aligned = aligned_to(out, 16);
    if (!aligned_to(out, dtype_size(out_dtype))) return refuse_reduce(fail(LBC_EINVAL, "out is not aligned to its element size"));
    for (int r = 0; r < world; ++r) {
        if (codes[r] == nullptr || scales[r] == nullptr) return refuse_reduce(fail(LBC_EINVAL, "payload %d has a null pointer", r));
        if (!aligned_to(scales[r], 4)) return refuse_reduce(fail(LBC_EINVAL, "scales of payload %d must be 4-byte aligned", r));
        aligned = aligned && aligned_to(codes[r], vec);
        c.args.codes[r] = codes[r];
        c.args.scales[r] = scales[r];
    }
    if (prepared != nullptr) {
        if (!aligned_to(prepared, dtype_size(out_dtype)) || !aligned_to(new_residual, dtype_size(out_dtype)))
            return refuse_reduce(fail(LBC_EINVAL, "prepared/new_residual are not aligned to their element size"));
        aligned = aligned && aligned_to(prepared, 16) && aligned_to(new_residual, 16);
    }
    c.args.out = out;
    c.args.prepared = prepared;
    c.args.new_residual = new_residual;
    c.args.numel = numel;
    c.args.divisor = divisor;
    c.out_dtype = out_dtype;
    c.world = world;
    c.group_size = group_size;
    c.aligned = aligned;
    return c;
}

// Validation of lbc_dequant_reduce_quant, shared with the pipeline step.
ReduceQuantCall prepare_reduce_quant(const int8_t *const *codes, const float *const *scales, int world, int64_t numel,
                                     int group_size, float divisor, int mid_dtype, int8_t *out_codes, float *out_scales) {
    if (world <= 0) return refuse_reduce_quant(fail(LBC_EINVAL, "inputs must not be empty"));
    if (numel < 0) return refuse_reduce_quant(fail(LBC_EINVAL, "numel must be >= 0"));
    if (!(divisor > 0.0f)) return refuse_reduce_quant(fail(LBC_EINVAL, "divisor must be > 0"));
    if (!valid_dtype(mid_dtype)) return refuse_reduce_quant(fail(LBC_EINVAL, "unsupported intermediate dtype %d", mid_dtype));
    if (world > LBC_MAX_PAYLOADS || !valid_group(group_size)) return refuse_reduce_quant(LBC_UNSUPPORTED);
    ReduceQuantCall c;
    if (numel == 0) {
        c.empty = true;
        return c;
    }
    if (codes == nullptr || scales == nullptr || out_codes == nullptr || out_scales == nullptr)
        return refuse_reduce_quant(fail(LBC_EINVAL, "codes, scales, out_codes and out_scales must not be null"));
    if (!aligned_to(out_scales, 4)) return refuse_reduce_quant(fail(LBC_EINVAL, "out_scales must be 4-byte aligned"));
    bool aligned = aligned_to(out_codes, 4);
    for (int r = 0; r < world; ++r) {
        if (codes[r] == nullptr || scales[r] == nullptr) return refuse_reduce_quant(fail(LBC_EINVAL, "payload %d has a null pointer", r));
        if (!aligned_to(scales[r], 4)) return refuse_reduce_quant(fail(LBC_EINVAL, "scales of payload %d must be 4-byte aligned", r));
        if (codes[r] == out_codes || scales[r] == out_scales)
            return refuse_reduce_quant(fail(LBC_EINVAL, "the output payload must not alias input payload %d", r));
        aligned = aligned && aligned_to(codes[r], 4);
        c.args.codes[r] = codes[r];
        c.args.scales[r] = scales[r];
    }
    c.args.out_codes = out_codes;
    c.args.out_scales = out_scales;
    c.args.numel = numel;
    c.args.divisor = divisor;
    c.mid_dtype = mid_dtype;
    c.world = world;
    c.aligned = aligned;
    return c;
}

// Validation of lbc_dequant_chunks, shared in the same way.
DecodeCall prepare_decode_chunks(const uint8_t *payloads, int64_t payload_stride, int world, int64_t shard_numel,
                                 int64_t total_numel, int group_size, void *out, int out_dtype) {
    if (shard_numel < 0 || total_numel < 0) return refuse_decode(fail(LBC_EINVAL, "element counts must be >= 0"));
    if (world <= 0) return refuse_decode(fail(LBC_EINVAL, "world must be > 0"));
    if (total_numel > shard_numel * world) return refuse_decode(fail(LBC_EINVAL, "total_numel exceeds world * shard_numel"));
    if (!valid_dtype(out_dtype)) return refuse_decode(fail(LBC_EINVAL, "unsupported output dtype %d", out_dtype));
    if (!valid_group(group_size)) return refuse_decode(LBC_UNSUPPORTED);
    if (world > 65535) return refuse_decode(LBC_UNSUPPORTED);
    DecodeCall c;
    if (shard_numel == 0 || total_numel == 0) {
        c.empty = true;
        return c;
    }
    const int64_t groups = (shard_numel + group_size - 1) / group_size;
    const int64_t payload_bytes = groups * (group_size + 4);
    if (payloads == nullptr || out == nullptr) return refuse_decode(fail(LBC_EINVAL, "payloads and out must not be null"));
    if (payload_stride < payload_bytes || (payload_stride & 3) != 0)
        return refuse_decode(fail(LBC_EINVAL, "payload_stride must be a multiple of 4 and >= %lld", (long long)payload_bytes));
    if (!aligned_to(payloads, 4)) return refuse_decode(fail(LBC_EINVAL, "payloads must be 4-byte aligned"));
    if (!aligned_to(out, dtype_size(out_dtype))) return refuse_decode(fail(LBC_EINVAL, "out is not aligned to its element size"));
    const int vec = out_dtype == LBC_F32 ? 4 : 8;
    c.aligned = aligned_to(payloads, vec) && payload_stride % vec == 0 && aligned_to(out, 16) &&
                (shard_numel * dtype_size(out_dtype)) % 16 == 0;
    c.args.codes_base = payloads;
    c.args.scales_base = payloads + groups * group_size;
    c.args.out = out;
    c.args.shard_numel = shard_numel;
    c.args.total_numel = total_numel;
    c.args.payload_stride = payload_stride;
    c.out_dtype = out_dtype;
    c.world = world;
    return c;
}

int launch_reduce(const ReduceCall &c, int access, void *stream) {
    if (c.status != LBC_OK || c.empty) return c.status;
    return finish(lbc::launch_dequant_reduce(c.out_dtype, c.group_size, c.world,
                                             pick_mode(c.aligned, access, c.args.numel * dtype_size(c.out_dtype)), c.args,
                                             static_cast<hipStream_t>(stream)),
                  "lbc_dequant_reduce");
}

}  // namespace

extern "C" {

int lbc_abi_version(void) { return LBC_ABI_VERSION; }

const char *lbc_last_error(void) { return g_error; }

int lbc_quant_pack(const void *x, int x_dtype, const void *residual, int residual_dtype, int64_t numel,
                   int group_size, int8_t *codes, float *scales, void *new_residual, int new_residual_dtype,
                   void *restored, int restored_dtype, void *prepared, int prepared_dtype, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    if (numel < 0) return fail(LBC_EINVAL, "numel must be >= 0");
    if (!valid_dtype(x_dtype)) return fail(LBC_EINVAL, "unsupported input dtype %d", x_dtype);
    if (residual != nullptr && !valid_dtype(residual_dtype))
        return fail(LBC_EINVAL, "unsupported residual dtype %d", residual_dtype);
    if (!valid_group(group_size)) return LBC_UNSUPPORTED;
    if (numel == 0) return LBC_OK;
    if (x == nullptr) return fail(LBC_EINVAL, "input must not be null");
    if (codes == nullptr || scales == nullptr) return fail(LBC_EINVAL, "codes and scales must not be null");
    if (!aligned_to(scales, 4)) return fail(LBC_EINVAL, "scales must be 4-byte aligned");
    if (!aligned_to(x, dtype_size(x_dtype))) return fail(LBC_EINVAL, "input is not aligned to its element size");
    return launch_quant(quant_pack_common(x, x_dtype, residual, residual_dtype, numel, 1, group_size,
                                          reinterpret_cast<uint8_t *>(codes), reinterpret_cast<uint8_t *>(scales), 0, numel,
                                          new_residual, new_residual_dtype, restored, restored_dtype, prepared, prepared_dtype),
                        "lbc_quant_pack", access, stream);
}

int lbc_quant_pack_chunks(const void *x, int x_dtype, const void *residual, int residual_dtype, int64_t numel,
                          int world, int group_size, uint8_t *payloads, int64_t payload_stride, void *new_residual,
                          int new_residual_dtype, void *restored, int restored_dtype, void *prepared, int prepared_dtype,
                          int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    return launch_quant(prepare_quant_chunks(x, x_dtype, residual, residual_dtype, numel, world, group_size, payloads,
                                             payload_stride, new_residual, new_residual_dtype, restored, restored_dtype,
                                             prepared, prepared_dtype),
                        "lbc_quant_pack_chunks", access, stream);
}

int lbc_dequant(const int8_t *codes, const float *scales, int64_t numel, int group_size, void *out,
                int out_dtype, int reduce_op, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    if (numel < 0) return fail(LBC_EINVAL, "numel must be >= 0");
    if (!valid_dtype(out_dtype)) return fail(LBC_EINVAL, "unsupported output dtype %d", out_dtype);
    if (reduce_op < LBC_REDUCE_NONE || reduce_op > LBC_REDUCE_MIN)
        return fail(LBC_EINVAL, "unsupported reduce op %d", reduce_op);
    if (!valid_group(group_size)) return LBC_UNSUPPORTED;
    if (numel == 0) return LBC_OK;
    if (codes == nullptr || scales == nullptr || out == nullptr)
        return fail(LBC_EINVAL, "codes, scales and out must not be null");
    if (!aligned_to(scales, 4)) return fail(LBC_EINVAL, "scales must be 4-byte aligned");
    if (!aligned_to(out, dtype_size(out_dtype))) return fail(LBC_EINVAL, "out is not aligned to its element size");
    const int vec = out_dtype == LBC_F32 ? 4 : 8;
    const bool aligned = aligned_to(codes, vec) && aligned_to(out, 16);
    lbc::DecodeArgs a{};
    a.codes_base = reinterpret_cast<const uint8_t *>(codes);
    a.scales_base = reinterpret_cast<const uint8_t *>(scales);
    a.out = out;
    a.shard_numel = numel;
    a.total_numel = numel;
    a.payload_stride = 0;
    return finish(lbc::launch_decode(out_dtype, group_size, reduce_op, pick_mode(aligned, access),
                                     a, 1, static_cast<hipStream_t>(stream)),
                  "lbc_dequant");
}

int lbc_dequant_chunks(const uint8_t *payloads, int64_t payload_stride, int world, int64_t shard_numel,
                       int64_t total_numel, int group_size, void *out, int out_dtype, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    const DecodeCall c = prepare_decode_chunks(payloads, payload_stride, world, shard_numel, total_numel, group_size, out,
                                               out_dtype);
    if (c.status != LBC_OK || c.empty) return c.status;
    return finish(lbc::launch_decode(c.out_dtype, group_size, LBC_REDUCE_NONE, pick_mode(c.aligned, access), c.args, c.world,
                                     static_cast<hipStream_t>(stream)),
                  "lbc_dequant_chunks");
}

int lbc_dequant_reduce(const int8_t *const *codes, const float *const *scales, int world, int64_t numel,
                       int group_size, float divisor, void *out, int out_dtype, const void *prepared,
                       void *new_residual, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    return launch_reduce(prepare_reduce(codes, scales, world, numel, group_size, divisor, out, out_dtype, prepared,
                                        new_residual),
                         access, stream);
}

int lbc_quant_pack_chunks_and_dequant_reduce(
    const void *x, int x_dtype, const void *residual, int residual_dtype, int64_t numel, int world, int group_size,
    uint8_t *payloads, int64_t payload_stride, void *new_residual, int new_residual_dtype,
    const int8_t *const *codes, const float *const *scales, int reduce_world, int64_t reduce_numel, float divisor,
    void *out, int out_dtype, const void *prepared, void *reduce_new_residual, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    const QuantCall q = prepare_quant_chunks(x, x_dtype, residual, residual_dtype, numel, world, group_size, payloads,
                                             payload_stride, new_residual, new_residual_dtype, nullptr, LBC_F32, nullptr,
                                             LBC_NONE);
    if (q.status != LBC_OK) return q.status;
    const ReduceCall r = prepare_reduce(codes, scales, reduce_world, reduce_numel, group_size, divisor, out, out_dtype,
                                        prepared, reduce_new_residual);
    if (r.status != LBC_OK) return r.status;
    if (q.empty) return launch_reduce(r, access, stream);
    if (r.empty) return launch_quant(q, "lbc_quant_pack_chunks_and_dequant_reduce", access, stream);
    // one grid exists for aligned operands, whole 16-byte chunks, group 64 and a residual that is absent or fp32;
    // everything else is for the caller to issue as the two separate calls
    if (!q.aligned || !r.aligned || group_size != 64 || (q.r_dtype != LBC_NONE && q.r_dtype != LBC_F32))
        return LBC_UNSUPPORTED;
    // the quantize half is the instantiation the separate call would run: its lane width also decided q.aligned
    const int vec = lbc::quant_pack_vec(q.x_dtype, q.r_dtype, q.d_dtype, q.outputs);
    return finish(lbc::launch_bucket_step(q.x_dtype, q.r_dtype, vec, r.out_dtype, r.world, pick_mode(true, access), q.args,
                                          q.world, r.args, static_cast<hipStream_t>(stream)),
                  "lbc_quant_pack_chunks_and_dequant_reduce");
}

int lbc_dequant_reduce_quant(const int8_t *const *codes, const float *const *scales, int world, int64_t numel,
                             int group_size, float divisor, int mid_dtype, int8_t *out_codes, float *out_scales, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    const ReduceQuantCall c = prepare_reduce_quant(codes, scales, world, numel, group_size, divisor, mid_dtype, out_codes,
                                                   out_scales);
    if (c.status != LBC_OK || c.empty) return c.status;
    return finish(lbc::launch_dequant_reduce_quant(c.mid_dtype, group_size, c.world, pick_mode(c.aligned, access), c.args,
                                                   static_cast<hipStream_t>(stream)),
                  "lbc_dequant_reduce_quant");
}

int lbc_bucket_pipeline_step(const lbc_quant_chunks_stage *quant, const lbc_reduce_quant_stage *reduce,
                             const lbc_dequant_chunks_stage *decode, int group_size, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    QuantCall q;
    q.empty = true;
    if (quant != nullptr) {
        q = prepare_quant_chunks(quant->x, quant->x_dtype, quant->residual, quant->residual_dtype, quant->numel, quant->world,
                                 group_size, quant->payloads, quant->payload_stride, quant->new_residual,
                                 quant->new_residual_dtype, nullptr, LBC_F32, nullptr, LBC_NONE);
        if (q.status != LBC_OK) return q.status;
    }
    ReduceQuantCall r;
    r.empty = true;
    if (reduce != nullptr) {
        r = prepare_reduce_quant(reduce->codes, reduce->scales, reduce->world, reduce->numel, group_size, reduce->divisor,
                                 reduce->mid_dtype, reduce->out_codes, reduce->out_scales);
        if (r.status != LBC_OK) return r.status;
    }
    DecodeCall d;
    d.empty = true;
    if (decode != nullptr) {
        d = prepare_decode_chunks(decode->payloads, decode->payload_stride, decode->world, decode->shard_numel,
                                  decode->total_numel, group_size, decode->out, decode->out_dtype);
        if (d.status != LBC_OK) return d.status;
    }
    const int stages = (q.empty ? 0 : 1) + (r.empty ? 0 : 1) + (d.empty ? 0 : 1);
    if (stages == 0) return LBC_OK;
    if (stages > 1) {
        // Nothing orders the stages inside the launch: what one writes, no other may read or write.
        struct Span { const char *low, *high; int stage; bool written; };
        Span spans[24];
        int count = 0;
        auto add = [&](const void *p, int64_t bytes, int stage, bool written) {
            if (p != nullptr && bytes > 0) spans[count++] = {static_cast<const char *>(p), static_cast<const char *>(p) + bytes, stage, written};
        };
        const int64_t groups_of_r = r.empty ? 0 : (reduce->numel + group_size - 1) / group_size;
        auto payload_bytes = [&](int64_t numel) { return (numel + group_size - 1) / group_size * (group_size + 4); };
        if (!q.empty) {
            add(quant->x, quant->numel * dtype_size(quant->x_dtype), 0, false);
            if (quant->residual != nullptr) add(quant->residual, quant->numel * dtype_size(quant->residual_dtype), 0, false);
            add(quant->payloads, (quant->world - 1) * quant->payload_stride + payload_bytes((quant->numel + quant->world - 1) / quant->world), 0, true);
            if (quant->new_residual != nullptr) add(quant->new_residual, quant->numel * dtype_size(quant->new_residual_dtype), 0, true);
        }
        if (!r.empty) {
            for (int i = 0; i < reduce->world; ++i) {
                add(reduce->codes[i], reduce->numel, 1, false);
                add(reduce->scales[i], groups_of_r * 4, 1, false);
            }
            add(reduce->out_codes, groups_of_r * group_size, 1, true);
            add(reduce->out_scales, groups_of_r * 4, 1, true);
        }
        if (!d.empty) {
            add(decode->payloads, (decode->world - 1) * decode->payload_stride + payload_bytes(decode->shard_numel), 2, false);
            add(decode->out, decode->total_numel * dtype_size(decode->out_dtype), 2, true);
        }
        for (int i = 0; i < count; ++i) {
            if (!spans[i].written) continue;
            for (int j = 0; j < count; ++j)
                if (spans[i].stage != spans[j].stage && spans[i].low < spans[j].high && spans[j].low < spans[i].high)
                    return fail(LBC_EINVAL, "a stage writes memory that another stage of the same launch reads or writes");
        }
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (stages == 1) {          // one stage with work: its own kernel
        if (!q.empty) return launch_quant(q, "lbc_bucket_pipeline_step", access, stream);
        if (!r.empty)
            return finish(lbc::launch_dequant_reduce_quant(r.mid_dtype, group_size, r.world, pick_mode(r.aligned, access), r.args, s),
                          "lbc_bucket_pipeline_step");
        return finish(lbc::launch_decode(d.out_dtype, group_size, LBC_REDUCE_NONE, pick_mode(d.aligned, access), d.args, d.world, s),
                      "lbc_bucket_pipeline_step");
    }
    // one grid exists for group 64, operands aligned for the vector kernels, a residual that is absent or fp32,
    // and one element type for the bucket, the reduce and the decoded output
    if (group_size != 64 || (!q.empty && !q.aligned) || (!r.empty && !r.aligned) || (!d.empty && !d.aligned))
        return LBC_UNSUPPORTED;
    if (!q.empty && q.r_dtype != LBC_NONE && q.r_dtype != LBC_F32) return LBC_UNSUPPORTED;
    const int dtype = !q.empty ? q.x_dtype : (!r.empty ? r.mid_dtype : d.out_dtype);
    if ((!r.empty && r.mid_dtype != dtype) || (!d.empty && d.out_dtype != dtype)) return LBC_UNSUPPORTED;
    const int vec = q.empty ? 4 : lbc::quant_pack_vec(q.x_dtype, q.r_dtype, q.d_dtype, q.outputs);
    return finish(lbc::launch_pipeline_step(dtype, q.empty ? LBC_NONE : q.r_dtype, vec, pick_mode(true, access),
                                            q.empty ? nullptr : &q.args, q.world, r.empty ? nullptr : &r.args, r.world,
                                            d.empty ? nullptr : &d.args, d.world, s),
                  "lbc_bucket_pipeline_step");
}

int lbc_ring_step(const int8_t *recv_codes, const float *recv_scales, void *chunk, int dtype, int64_t numel,
                  int group_size, int reduce_op, float divisor, int8_t *send_codes, float *send_scales, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    if (numel < 0) return fail(LBC_EINVAL, "numel must be >= 0");
    if (!valid_dtype(dtype)) return fail(LBC_EINVAL, "unsupported chunk dtype %d", dtype);
    if (reduce_op < LBC_REDUCE_NONE || reduce_op > LBC_REDUCE_MIN) return fail(LBC_EINVAL, "unknown reduce op %d", reduce_op);
    if (!(divisor > 0.0f)) return fail(LBC_EINVAL, "divisor must be > 0");
    if ((send_codes == nullptr) != (send_scales == nullptr))
        return fail(LBC_EINVAL, "send codes and send scales must be given together");
    if (!valid_group(group_size)) return LBC_UNSUPPORTED;
    if (reduce_op != LBC_REDUCE_NONE && reduce_op != LBC_REDUCE_SUM) return LBC_UNSUPPORTED;
    if (numel == 0) return LBC_OK;
    if (recv_codes == nullptr || recv_scales == nullptr) return fail(LBC_EINVAL, "received codes and scales must not be null");
    if (chunk == nullptr) return fail(LBC_EINVAL, "chunk must not be null");
    if (!aligned_to(chunk, dtype_size(dtype))) return fail(LBC_EINVAL, "chunk is not aligned to its element size");
    if (!aligned_to(recv_scales, 4) || (send_scales != nullptr && !aligned_to(send_scales, 4)))
        return fail(LBC_EINVAL, "scales must be 4-byte aligned");
    if (send_codes == recv_codes || send_scales == recv_scales)
        return fail(LBC_EINVAL, "the payload to send must not alias the received one");
    const int vec = 16 / dtype_size(dtype);   // elements, and code bytes, one lane owns
    const bool aligned = aligned_to(chunk, 16) && aligned_to(recv_codes, vec) &&
                         (send_codes == nullptr || aligned_to(send_codes, vec));
    lbc::RingStepArgs a{recv_codes, recv_scales, chunk, send_codes, send_scales, numel, divisor};
    return finish(lbc::launch_ring_step(dtype, group_size, reduce_op == LBC_REDUCE_SUM, pick_mode(aligned, access), a,
                                        static_cast<hipStream_t>(stream)),
                  "lbc_ring_step");
}

int lbc_ef_update(const void *prepared, int prepared_dtype, const void *restored, int restored_dtype,
                  void *residual, int residual_dtype, int64_t numel, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    if (numel < 0) return fail(LBC_EINVAL, "numel must be >= 0");
    if (!valid_dtype(prepared_dtype) || !valid_dtype(restored_dtype) || !valid_dtype(residual_dtype))
        return fail(LBC_EINVAL, "unsupported dtype");
    if (numel == 0) return LBC_OK;
    if (prepared == nullptr || restored == nullptr || residual == nullptr)
        return fail(LBC_EINVAL, "prepared, restored and residual must not be null");
    if (!aligned_to(prepared, dtype_size(prepared_dtype)) || !aligned_to(restored, dtype_size(restored_dtype)) ||
        !aligned_to(residual, dtype_size(residual_dtype)))
        return fail(LBC_EINVAL, "a tensor is not aligned to its element size");
    const bool aligned = aligned_to(prepared, 16) && aligned_to(restored, 16) && aligned_to(residual, 16);
    lbc::EfArgs a{prepared, restored, residual, numel};
    return finish(lbc::launch_ef_update(prepared_dtype, restored_dtype, residual_dtype, pick_mode(aligned, access), a,
                                        static_cast<hipStream_t>(stream)),
                  "lbc_ef_update");
}

// ---- payload format of the reference's CUDA extension -------------------------------------
int64_t lbc_wire_payload_nbytes(int64_t numel, int group_size, int dtype, int bit) {
    if (numel < 0 || !valid_group(group_size) || !valid_dtype(dtype) || (bit != 8 && bit != 4)) return -1;
    const int64_t groups = numel == 0 ? 0 : (numel + group_size - 1) / group_size;
    return groups * (group_size * bit / 8 + dtype_size(dtype));
}

int lbc_wire_quant_pack_chunks(const void *x, const void *residual, int dtype, int64_t numel, int world,
                               int group_size, int bit, int compact, uint8_t *payloads, int64_t payload_stride, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    if (numel < 0) return fail(LBC_EINVAL, "numel must be >= 0");
    if (world <= 0) return fail(LBC_EINVAL, "world must be > 0");
    if (!valid_dtype(dtype)) return fail(LBC_EINVAL, "unsupported dtype %d", dtype);
    if (!valid_group(group_size) || world > 65535 || (bit != 8 && bit != 4)) return LBC_UNSUPPORTED;
    const int64_t shard = (numel + world - 1) / world;
    if (shard == 0) return LBC_OK;
    const int item = dtype_size(dtype);
    const int64_t payload_bytes = lbc_wire_payload_nbytes(shard, group_size, dtype, bit);
    if (x == nullptr || payloads == nullptr) return fail(LBC_EINVAL, "input and payloads must not be null");
    if (world > 1 && (payload_stride < payload_bytes || payload_stride % item != 0))
        return fail(LBC_EINVAL, "payload_stride must be a multiple of %d and >= %lld", item, (long long)payload_bytes);
    if (!aligned_to(payloads, item)) return fail(LBC_EINVAL, "payloads must be aligned to the element size");
    if (!aligned_to(x, item) || !aligned_to(residual, item))
        return fail(LBC_EINVAL, "input/residual are not aligned to their element size");
    lbc::WireQuantArgs a{};
    a.x = x;
    a.residual = residual;
    a.payloads = payloads;
    a.numel = numel;
    a.shard_numel = shard;
    a.payload_stride = world > 1 ? payload_stride : 0;
    a.compact = compact != 0;
    a.nan_resets = residual == nullptr;
    return finish(lbc::launch_wire_quant(dtype, group_size, bit, pick_mode(true, access), a, world,
                                         static_cast<hipStream_t>(stream)),
                  "lbc_wire_quant_pack");
}

int lbc_wire_quant_pack(const void *x, const void *residual, int dtype, int64_t numel, int group_size, int bit,
                        int compact, uint8_t *payload, int access, void *stream) {
    return lbc_wire_quant_pack_chunks(x, residual, dtype, numel, 1, group_size, bit, compact, payload, 0, access, stream);
}

int lbc_wire_dequant_chunks(const uint8_t *payloads, int64_t payload_stride, int world, int64_t shard_numel,
                            int64_t total_numel, int group_size, int bit, int compact, void *out, int dtype,
                            int reduce_op, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    if (shard_numel < 0 || total_numel < 0) return fail(LBC_EINVAL, "element counts must be >= 0");
    if (world <= 0) return fail(LBC_EINVAL, "world must be > 0");
    if (total_numel > shard_numel * world) return fail(LBC_EINVAL, "total_numel exceeds world * shard_numel");
    if (!valid_dtype(dtype)) return fail(LBC_EINVAL, "unsupported dtype %d", dtype);
    if (reduce_op < LBC_REDUCE_NONE || reduce_op > LBC_REDUCE_MIN)
        return fail(LBC_EINVAL, "unsupported reduce op %d", reduce_op);
    if (!valid_group(group_size) || world > 65535 || (bit != 8 && bit != 4)) return LBC_UNSUPPORTED;
    if (shard_numel == 0 || total_numel == 0) return LBC_OK;
    const int item = dtype_size(dtype);
    const int64_t payload_bytes = lbc_wire_payload_nbytes(shard_numel, group_size, dtype, bit);
    if (payloads == nullptr || out == nullptr) return fail(LBC_EINVAL, "payloads and out must not be null");
    if (world > 1 && (payload_stride < payload_bytes || payload_stride % item != 0))
        return fail(LBC_EINVAL, "payload_stride must be a multiple of %d and >= %lld", item, (long long)payload_bytes);
    if (!aligned_to(payloads, item) || !aligned_to(out, item))
        return fail(LBC_EINVAL, "payloads/out must be aligned to the element size");
    lbc::WireDecodeArgs a{};
    a.payloads = payloads;
    a.out = out;
    a.shard_numel = shard_numel;
    a.total_numel = total_numel;
    a.payload_stride = world > 1 ? payload_stride : 0;
    a.compact = compact != 0;
    return finish(lbc::launch_wire_decode(dtype, group_size, bit, reduce_op, pick_mode(true, access), a, world,
                                          static_cast<hipStream_t>(stream)),
                  "lbc_wire_dequant");
}

int lbc_wire_dequant(const uint8_t *payload, int64_t numel, int group_size, int bit, int compact, void *out,
                     int dtype, int reduce_op, int access, void *stream) {
    return lbc_wire_dequant_chunks(payload, 0, 1, numel, numel, group_size, bit, compact, out, dtype, reduce_op,
                                   access, stream);
}

int lbc_wire_dequant_reduce(const uint8_t *const *payloads, int world, int64_t numel, int group_size, int compact,
                            float inv_divisor, int fused_multiply_add, void *out, int dtype, const void *prepared,
                            void *new_residual, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    if (world <= 0) return fail(LBC_EINVAL, "inputs must not be empty");
    if (numel < 0) return fail(LBC_EINVAL, "numel must be >= 0");
    if (!(inv_divisor > 0.0f)) return fail(LBC_EINVAL, "inv_divisor must be > 0");
    if (!valid_dtype(dtype)) return fail(LBC_EINVAL, "unsupported dtype %d", dtype);
    if ((prepared == nullptr) != (new_residual == nullptr))
        return fail(LBC_EINVAL, "prepared and new_residual must be given together");
    if (world > LBC_MAX_PAYLOADS || group_size != 64) return LBC_UNSUPPORTED;
    if (numel == 0) return LBC_OK;
    if (payloads == nullptr || out == nullptr) return fail(LBC_EINVAL, "payloads and out must not be null");
    const int item = dtype_size(dtype);
    if (!aligned_to(out, item) || !aligned_to(prepared, item) || !aligned_to(new_residual, item))
        return fail(LBC_EINVAL, "out/prepared/new_residual are not aligned to their element size");
    lbc::WireReduceArgs a{};
    for (int r = 0; r < world; ++r) {
        if (payloads[r] == nullptr) return fail(LBC_EINVAL, "payload %d is null", r);
        if (!aligned_to(payloads[r], item)) return fail(LBC_EINVAL, "payload %d must be aligned to the element size", r);
        a.payloads[r] = payloads[r];
    }
    a.out = out;
    a.prepared = prepared;
    a.new_residual = new_residual;
    a.numel = numel;
    a.inv_divisor = inv_divisor;
    a.compact = compact != 0;
    return finish(lbc::launch_wire_reduce(dtype, group_size, world, fused_multiply_add != 0, pick_mode(true, access), a,
                                          static_cast<hipStream_t>(stream)),
                  "lbc_wire_dequant_reduce");
}

int lbc_wire_ring_step(const uint8_t *received, void *chunk, int dtype, int64_t numel, int group_size, int compact,
                       int reduce_op, float divisor, uint8_t *send, int access, void *stream) {
    if (!valid_access(access)) return fail(LBC_EINVAL, "unknown access mode %d", access);
    if (numel < 0) return fail(LBC_EINVAL, "numel must be >= 0");
    if (!valid_dtype(dtype)) return fail(LBC_EINVAL, "unsupported chunk dtype %d", dtype);
    if (reduce_op < LBC_REDUCE_NONE || reduce_op > LBC_REDUCE_MIN) return fail(LBC_EINVAL, "unknown reduce op %d", reduce_op);
    if (!(divisor > 0.0f)) return fail(LBC_EINVAL, "divisor must be > 0");
    if (!valid_group(group_size)) return LBC_UNSUPPORTED;
    if (reduce_op != LBC_REDUCE_NONE && reduce_op != LBC_REDUCE_SUM) return LBC_UNSUPPORTED;
    if (numel % group_size != 0) return fail(LBC_EINVAL, "numel should be multiple of group_size");
    if (numel == 0) return LBC_OK;
    if (received == nullptr || chunk == nullptr) return fail(LBC_EINVAL, "received payload and chunk must not be null");
    const int item = dtype_size(dtype);
    if (!aligned_to(chunk, item) || !aligned_to(received, item) || !aligned_to(send, item))
        return fail(LBC_EINVAL, "chunk and payloads must be aligned to the element size");
    if (send == received) return fail(LBC_EINVAL, "the payload to send must not alias the received one");
    lbc::WireRingStepArgs a{received, chunk, send, numel, divisor == 1.0f ? 1.0f : 1.0f / divisor, compact != 0};
    return finish(lbc::launch_wire_ring_step(dtype, group_size, reduce_op == LBC_REDUCE_SUM, pick_mode(true, access), a,
                                             static_cast<hipStream_t>(stream)),
                  "lbc_wire_ring_step");
}

// ---- general policies of that format: code books, stochastic rounding, top-k ------------------
static bool valid_general(int group_size, int bit, int quant_type, int topk) {
    if (!valid_group(group_size) || (bit != 8 && bit != 4) || topk < 0 || topk > 2) return false;
    if (quant_type < LBC_QUANT_LINEAR || quant_type > LBC_QUANT_E2M1) return false;
    return quant_type == LBC_QUANT_LINEAR || bit == 4;
}

int64_t lbc_wire_general_payload_nbytes(int64_t numel, int group_size, int dtype, int bit, int topk) {
    if (numel < 0 || !valid_dtype(dtype) || !valid_general(group_size, bit, LBC_QUANT_LINEAR, topk)) return -1;
    const int64_t groups = numel == 0 ? 0 : (numel + group_size - 1) / group_size;
    return groups * (group_size * bit / 8 + dtype_size(dtype) * (topk == 0 ? 1 : topk + 2));
}

int lbc_wire_quant_general(const void *x, int dtype, int64_t numel, int group_size, int bit, int quant_type, int topk,
                           int stochastic, uint64_t seed, uint64_t offset, int compact, uint8_t *payload, void *stream) {
    if (numel < 0) return fail(LBC_EINVAL, "numel must be >= 0");
    if (!valid_dtype(dtype)) return fail(LBC_EINVAL, "unsupported dtype %d", dtype);
    if (!valid_general(group_size, bit, quant_type, topk)) return LBC_UNSUPPORTED;
    if (numel % group_size != 0) return fail(LBC_EINVAL, "input numel should be multiple of group_size");
    if (numel == 0) return LBC_OK;
    const int item = dtype_size(dtype);
    if (x == nullptr || payload == nullptr) return fail(LBC_EINVAL, "input and payload must not be null");
    if (!aligned_to(x, item) || !aligned_to(payload, item))
        return fail(LBC_EINVAL, "input/payload must be aligned to the element size");
    // Plain linear codes without outliers or noise are what the dedicated pack kernel writes (with the NaN rule of
    // the general kernels for a call without a residual): same bytes, a memory-bound kernel instead of this
    // instruction-bound one.
    if (quant_type == 0 && topk == 0 && stochastic == 0)
        return lbc_wire_quant_pack(x, nullptr, dtype, numel, group_size, bit, compact, payload, LBC_ACCESS_AUTO, stream);
    lbc::WireGeneralQuantArgs a{};
    a.x = x;
    a.payload = payload;
    a.numel = numel;
    a.kind = quant_type;
    a.topk = topk;
    a.stochastic = stochastic != 0;
    a.compact = compact != 0;
    a.seed = seed;
    a.offset = offset;
    return finish(lbc::launch_wire_general_quant(dtype, group_size, bit, a, static_cast<hipStream_t>(stream)),
                  "lbc_wire_quant_general");
}

int lbc_wire_dequant_general(const uint8_t *payload, int64_t numel, int group_size, int bit, int quant_type, int topk,
                             int compact, void *out, int dtype, int reduce_op, void *stream) {
    if (numel < 0) return fail(LBC_EINVAL, "numel must be >= 0");
    if (!valid_dtype(dtype)) return fail(LBC_EINVAL, "unsupported dtype %d", dtype);
    if (reduce_op < LBC_REDUCE_NONE || reduce_op > LBC_REDUCE_MIN)
        return fail(LBC_EINVAL, "unsupported reduce op %d", reduce_op);
    if (!valid_general(group_size, bit, quant_type, topk)) return LBC_UNSUPPORTED;
    if (numel % group_size != 0) return fail(LBC_EINVAL, "numel should be multiple of group_size");
    if (numel == 0) return LBC_OK;
    const int item = dtype_size(dtype);
    if (payload == nullptr || out == nullptr) return fail(LBC_EINVAL, "payload and out must not be null");
    if (!aligned_to(payload, item) || !aligned_to(out, item))
        return fail(LBC_EINVAL, "payload/out must be aligned to the element size");
    // Linear codes without an outlier channel decode the same way however they were rounded: the dedicated decode
    // kernel reads the same bytes at the memory-bound rate.
    if (quant_type == 0 && topk == 0)
        return lbc_wire_dequant(payload, numel, group_size, bit, compact, out, dtype, reduce_op, LBC_ACCESS_AUTO, stream);
    lbc::WireGeneralDecodeArgs a{};
    a.payload = payload;
    a.out = out;
    a.numel = numel;
    a.kind = quant_type;
    a.topk = topk;
    a.compact = compact != 0;
    a.op = reduce_op;
    return finish(lbc::launch_wire_general_decode(dtype, group_size, bit, a, static_cast<hipStream_t>(stream)),
                  "lbc_wire_dequant_general");
}

}  // extern "C"
