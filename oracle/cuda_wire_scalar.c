/*
 * Scalar C restatement of the reference's CUDA wire format.  TEST INFRASTRUCTURE ONLY.
 *
 * One element at a time, reading and writing payload bytes at the offsets the
 * reference kernels compute, with hand-written fp16/bf16 conversions so that
 * nothing is shared with the numpy restatement.  Compiled with
 * -ffp-contract=off; the fused multiply-add variant of the reduce calls fmaf
 * explicitly.  The product never links this file.
 *
 * Reference lines followed (paths under the upstream repository):
 *   lbw_quantize    ccdl_comm/csrc/quantization/quant_pack_kernel.cu:45-162
 *                   (non-compact offsets: quant_kernel_fp32.cuh:266-303)
 *   lbw_dequantize  ccdl_comm/csrc/quantization/dequant_kernel_fp32.cuh:81-120,
 *                   dequant_kernel.cuh:15-60
 *   lbw_reduce      ccdl_comm/csrc/quantization/dequant_reduce_kernel.cu:27-134,150-221
 *
 * dtype: 0 fp32, 1 fp16, 2 bf16 (16-bit values travel as uint16 bit patterns).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#include "scalar_floats.h"

enum { LBW_F32 = 0, LBW_F16 = 1, LBW_BF16 = 2 };

static int item_size(int dtype) { return dtype == LBW_F32 ? 4 : 2; }

static float load_as_f32(const void *base, int64_t index, int dtype) {
    if (dtype == LBW_F32) return ((const float *)base)[index];
    uint16_t h = ((const uint16_t *)base)[index];
    return dtype == LBW_F16 ? f16_to_f32(h) : bf16_to_f32(h);
}

static float round_to(float v, int dtype) {
    if (dtype == LBW_F16) return f16_to_f32(f32_to_f16(v));
    if (dtype == LBW_BF16) return bf16_to_f32(f32_to_bf16(v));
    return v;
}

static void store_from_f32(void *base, int64_t index, int dtype, float v) {
    if (dtype == LBW_F32) ((float *)base)[index] = v;
    else ((uint16_t *)base)[index] = dtype == LBW_F16 ? f32_to_f16(v) : f32_to_bf16(v);
}

static int64_t group_count(int64_t numel, int g) { return numel ? (numel + g - 1) / g : 0; }
/* cb = code bytes per group (g for 8-bit codes, g/2 for 4-bit codes) */
static int64_t code_offset(int64_t group, int cb, int item, int compact) {
    return compact ? group * (cb + item) : group * cb;
}
static int64_t scale_offset(int64_t group, int64_t groups, int cb, int item, int compact) {
    return compact ? group * (cb + item) + cb : groups * cb + group * item;
}

/* position of element k of a group inside the group's code bytes */
static int byte_slot(int k, int item) { return (k / item) * item + (item - 1 - k % item); }

/* 4-bit codes: element k of a group lives in a word of `item` bytes holding 2*item elements, first element in
 * the most significant nibble; the word is stored little-endian (quant_pack_kernel.cu:120-130,145-158). */
static int nibble_byte(int k, int item) {
    const int per_word = 2 * item;
    const int in_word = k % per_word;
    return (k / per_word) * item + (item - 1 - in_word / 2);
}
static int nibble_is_high(int k) { return (k % 2) == 0; }

void lbw_quantize(const void *x, const void *residual, int dtype, int64_t numel, int g, int compact, int bit,
                  uint8_t *payload) {
    const int item = item_size(dtype);
    const int cb = g * bit / 8;
    const float levels = bit == 8 ? 127.0f : 7.0f;
    const int64_t groups = group_count(numel, g);
    float prepared[256];
    for (int64_t group = 0; group < groups; ++group) {
        float max_abs = 0.0f;
        for (int k = 0; k < g; ++k) {
            const int64_t e = group * g + k;
            float v = 0.0f;
            if (e < numel) {
                v = load_as_f32(x, e, dtype);
                if (residual) v = round_to(v + load_as_f32(residual, e, dtype), dtype);
            }
            prepared[k] = v;
            max_abs = fmaxf(max_abs, fabsf(v));
        }
        const float stored = round_to(max_abs, dtype);
        const float scale = fmaxf(stored, 1.0e-6f);
        const float multiplier = levels / scale;
        uint8_t *codes = payload + code_offset(group, cb, item, compact);
        if (bit == 4) memset(codes, 0, (size_t)cb);
        for (int k = 0; k < g; ++k) {
            float q = rintf(prepared[k] * multiplier);
            int c = q != q ? 0 : (q > levels ? (int)levels : (q < -levels ? -(int)levels : (int)q));
            if (bit == 8) codes[byte_slot(k, item)] = (uint8_t)(int8_t)c;
            else codes[nibble_byte(k, item)] |= (uint8_t)((c & 0xF) << (nibble_is_high(k) ? 4 : 0));
        }
        uint8_t *where = payload + scale_offset(group, groups, cb, item, compact);
        if (dtype == LBW_F32) memcpy(where, &stored, 4);
        else {
            uint16_t h = dtype == LBW_F16 ? f32_to_f16(stored) : f32_to_bf16(stored);
            memcpy(where, &h, 2);
        }
    }
}

static float payload_step(const uint8_t *payload, int64_t group, int64_t groups, int g, int dtype, int compact,
                          int bit) {
    const int item = item_size(dtype);
    const uint8_t *where = payload + scale_offset(group, groups, g * bit / 8, item, compact);
    float stored;
    if (dtype == LBW_F32) memcpy(&stored, where, 4);
    else {
        uint16_t h;
        memcpy(&h, where, 2);
        stored = dtype == LBW_F16 ? f16_to_f32(h) : bf16_to_f32(h);
    }
    return stored / (bit == 8 ? 127.0f : 7.0f);
}

static float payload_code(const uint8_t *payload, int64_t e, int g, int dtype, int compact, int bit) {
    const int item = item_size(dtype);
    const int64_t group = e / g;
    const int k = (int)(e - group * g);
    const uint8_t *codes = payload + code_offset(group, g * bit / 8, item, compact);
    if (bit == 8) return (float)(int8_t)codes[byte_slot(k, item)];
    int nibble = (codes[nibble_byte(k, item)] >> (nibble_is_high(k) ? 4 : 0)) & 0xF;
    return (float)(nibble >= 8 ? nibble - 16 : nibble);
}

/* correctly rounded a + b in a 16-bit dtype: the double sum is exact (or, for far-apart bf16 operands,
 * off by far less than the rounding step) and is rounded once */
static float add_in_dtype(float a, float b, int dtype) {
    if (dtype == LBW_F32) return a + b;
    double wide = (double)a + (double)b;
    float near = (float)wide;
    double err = wide - (double)near;
    if (err != 0.0 && isfinite(near)) {
        uint32_t u = f32_to_bits(near);
        if ((u & 1u) == 0) {
            int up = (err > 0.0) == (near > 0.0f);
            u = up ? u + 1u : u - 1u;
            near = bits_to_f32(u);
        }
    }
    return round_to(near, dtype);
}

/* op: 0 none, 1 sum, 2 max, 3 min; out is read for op != 0 */
void lbw_dequantize(const uint8_t *payload, int64_t numel, int g, int compact, int dtype, int op, int bit,
                    void *out) {
    const int64_t groups = group_count(numel, g);
    for (int64_t e = 0; e < numel; ++e) {
        const float step = payload_step(payload, e / g, groups, g, dtype, compact, bit);
        float v = round_to(payload_code(payload, e, g, dtype, compact, bit) * step, dtype);
        if (op != 0) {
            const float old = load_as_f32(out, e, dtype);
            if (op == 1) v = add_in_dtype(old, v, dtype);
            else if (op == 2) v = old > v ? old : v;
            else v = old > v ? v : old;
        }
        store_from_f32(out, e, dtype, v);
    }
}

/* out = T(sum_r code_r * step_r * inv_divisor); with `prepared`, residual = T(prepared - unrounded mean) */
void lbw_reduce(const uint8_t *const *payloads, int world, int64_t numel, int g, int compact, int dtype,
                float inv_divisor, int use_fma, const void *prepared, void *out, void *residual) {
    const int64_t groups = group_count(numel, g);
    for (int64_t e = 0; e < numel; ++e) {
        float sum = 0.0f;
        for (int r = 0; r < world; ++r) {
            const float step = payload_step(payloads[r], e / g, groups, g, dtype, compact, 8);
            const float code = payload_code(payloads[r], e, g, dtype, compact, 8);
            if (use_fma) sum = fmaf(code, step, sum);
            else {
                const float term = code * step;
                sum = sum + term;
            }
        }
        const float value = sum * inv_divisor;
        store_from_f32(out, e, dtype, value);
        if (prepared && residual) store_from_f32(residual, e, dtype, load_as_f32(prepared, e, dtype) - value);
    }
}
