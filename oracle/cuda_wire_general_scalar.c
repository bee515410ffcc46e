/*
 * Scalar C restatement of the general quantize / dequantize kernels of the reference's CUDA
 * extension: non-linear 4-bit code books, stochastic rounding, the top-k side channel, the
 * NaN-resetting group maximum and the rotated scan of 16-bit groups.  TEST INFRASTRUCTURE ONLY.
 *
 * One group at a time, in the order the reference's one-thread-per-group kernels visit the
 * elements, writing and reading payload bytes at the offsets those kernels compute.  Compiled
 * with -ffp-contract=off; the one contraction nvcc applies by default (v * m + noise of the
 * stochastic linear encoder) is an explicit fmaf.  The product never links this file.
 *
 * Reference lines followed (paths under the upstream repository, ccdl_comm/csrc/quantization/):
 *   scale and top-k of a group   quant_kernel_fp32.cuh:87-165, quant_kernel.cuh:25-106
 *   encoder                      quant_kernel_fp32.cuh:168-205, quant_kernel.cuh:108-153, inner.cuh:44-97
 *   Philox stream                curand_init / curand / curand_uniform of cuRAND's Philox4_32_10
 *                                generator, seeded as quant_kernel_fp32.cuh:170-174
 *   layout                       quant_kernel_fp32.cuh:283-331 (appended), :390-445 (compact)
 *   decoder                      dequant_kernel_fp32.cuh:81-120,171-216, dequant_kernel.cuh:15-60, inner.cuh:67-72,118-138
 *   max / min with the output    utils.cuh:11-14
 *
 * dtype: 0 fp32, 1 fp16, 2 bf16.  kind: 0 linear, 1 normal, 2 uniform, 3 e3m0, 4 e2m1.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#include "scalar_floats.h"

enum { G_F32 = 0, G_F16 = 1, G_BF16 = 2 };

static const float BOOKS[4][16] = {
    {-1.0f, -0.815410147f, -0.655160150f, -0.510228027f, -0.375324982f, -0.246951370f, -0.122538030f, 0.0f,
     0.122538030f, 0.246951370f, 0.375324982f, 0.510228027f, 0.655160150f, 0.815410147f, 1.0f, INFINITY},
    {-1.0f, -0.85714286f, -0.71428571f, -0.57142857f, -0.42857143f, -0.28571429f, -0.14285714f, 0.0f,
     0.14285714f, 0.28571429f, 0.42857143f, 0.57142857f, 0.71428571f, 0.85714286f, 1.0f, INFINITY},
    {-1.0f, -0.5f, -0.25f, -0.125f, -0.0625f, -0.03125f, -0.015625f, 0.0f,
     0.015625f, 0.03125f, 0.0625f, 0.125f, 0.25f, 0.5f, 1.0f, INFINITY},
    {-1.0f, -0.6666666666666666f, -0.5f, -0.3333333333333333f, -0.25f, -0.16666666666666666f, -0.125f, 0.0f,
     0.125f, 0.16666666666666666f, 0.25f, 0.3333333333333333f, 0.5f, 0.6666666666666666f, 1.0f, INFINITY},
};

/* ---- Philox4x32-10 and the cuRAND state machine on top of it ------------------------------- */
typedef struct { uint32_t c[4], k[2], out[4]; int next; } philox_state;

static void philox_block(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
    for (int round = 0; round < 10; ++round) {
        if (round) { k0 += 0x9E3779B9u; k1 += 0xBB67AE85u; }
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

static void counter_add(uint32_t c[4], uint64_t n, int first_word) {   /* 128-bit counter += n << (32 * first_word) */
    uint64_t carry = n;
    for (int w = first_word; w < 4 && carry; ++w) {
        const uint64_t sum = (uint64_t)c[w] + (carry & 0xFFFFFFFFu);
        c[w] = (uint32_t)sum;
        carry = (carry >> 32) + (sum >> 32);
    }
}

static void stream_init(philox_state *s, uint64_t seed, uint64_t subsequence, uint64_t offset) {
    memset(s, 0, sizeof *s);
    s->k[0] = (uint32_t)seed;
    s->k[1] = (uint32_t)(seed >> 32);
    counter_add(s->c, subsequence, 2);          /* skipahead_sequence: the upper 64 bits */
    s->next = (int)(offset & 3);                /* skipahead: whole blocks, then words inside one */
    counter_add(s->c, offset >> 2, 0);
    philox_block(s->c, s->k, s->out);
}

static uint32_t stream_next(philox_state *s) {
    const uint32_t value = s->out[s->next++];
    if (s->next == 4) {
        counter_add(s->c, 1, 0);
        philox_block(s->c, s->k, s->out);
        s->next = 0;
    }
    return value;
}

static float stream_uniform(philox_state *s) {   /* (0, 1]: x * 2^-32 + 2^-33 */
    return (float)stream_next(s) * 0x1p-32f + 0x1p-33f;
}

/* exported for the known-answer tests */
void lbg_philox_block(const uint32_t *ctr, const uint32_t *key, uint32_t *out) { philox_block(ctr, key, out); }
void lbg_curand_draws(uint64_t seed, uint64_t subsequence, uint64_t offset, int count, uint32_t *out) {
    philox_state s;
    stream_init(&s, seed, subsequence, offset);
    for (int j = 0; j < count; ++j) out[j] = stream_next(&s);
}

/* ---- element access ------------------------------------------------------------------------ */
static int item_of(int dtype) { return dtype == G_F32 ? 4 : 2; }

static uint32_t raw_at(const void *base, int64_t index, int dtype) {
    if (dtype == G_F32) { uint32_t u; memcpy(&u, (const uint8_t *)base + 4 * index, 4); return u; }
    uint16_t h; memcpy(&h, (const uint8_t *)base + 2 * index, 2); return h;
}
static float raw_to_f32(uint32_t raw, int dtype) {
    if (dtype == G_F32) return bits_to_f32(raw);
    return dtype == G_F16 ? f16_to_f32((uint16_t)raw) : bf16_to_f32((uint16_t)raw);
}
static uint32_t f32_to_raw(float v, int dtype) {
    if (dtype == G_F32) return f32_to_bits(v);
    return dtype == G_F16 ? f32_to_f16(v) : f32_to_bf16(v);
}
static void put_word(uint8_t *where, uint32_t raw, int item) { memcpy(where, &raw, (size_t)item); }   /* little-endian host */
static uint32_t get_word(const uint8_t *where, int item) { uint32_t raw = 0; memcpy(&raw, where, (size_t)item); return raw; }

static int scan_start(int64_t group, int g, int dtype) {
    if (dtype == G_F32) return 0;
    const int banks = g / 4;
    return 4 * (int)((group & 31) / (32 / banks));
}
static int meta_words(int topk) { return topk == 0 ? 1 : topk + 2; }
static int64_t codes_at(int64_t group, int cb, int meta_bytes, int compact) {
    return compact ? group * (cb + meta_bytes) : group * cb;
}
static int64_t meta_at(int64_t group, int64_t groups, int cb, int meta_bytes, int compact) {
    return compact ? group * (cb + meta_bytes) + cb : groups * cb + group * meta_bytes;
}

/* ---- quantize ------------------------------------------------------------------------------ */
void lbg_quantize(const void *x, int dtype, int64_t numel, int g, int bit, int kind, int topk, int stochastic,
                  uint64_t seed, uint64_t offset, int compact, uint8_t *payload) {
    const int item = item_of(dtype), wide = dtype == G_F32;
    const int cb = g * bit / 8, mb = meta_words(topk) * item;
    const uint32_t sign_clear = wide ? 0x7FFFFFFFu : 0x7FFFu;
    const int64_t groups = numel / g;
    float v[256];
    uint32_t raw[256];
    for (int64_t group = 0; group < groups; ++group) {
        const int start = scan_start(group, g, dtype);
        for (int i = 0; i < g; ++i) {
            raw[i] = raw_at(x, group * g + i, dtype);
            v[i] = raw_to_f32(raw[i], dtype);
        }
        /* scale and top-k: running comparisons in scan order */
        float top1 = 0.0f, top2 = 0.0f, top3 = 0.0f;
        uint32_t bits1 = 0, bits2 = 0, bits3 = 0;
        int index1 = -1, index2 = -1;
        for (int j = 0; j < g; ++j) {
            const int i = (start + j) & (g - 1);
            const float a = fabsf(v[i]);
            const uint32_t a_bits = raw[i] & sign_clear;
            if (topk == 0) {
                if (!(top1 > a)) { top1 = a; bits1 = a_bits; }
                continue;
            }
            const int over1 = wide ? a >= top1 : a > top1;
            const int over2 = wide ? a >= top2 : a > top2;
            const int over3 = wide ? a >= top3 : a > top3;
            if (over1) {
                top3 = top2; bits3 = bits2;
                top2 = top1; bits2 = bits1; index2 = index1;
                top1 = a; bits1 = a_bits; index1 = i;
            } else if (over2) {
                top3 = top2; bits3 = bits2;
                top2 = a; bits2 = a_bits; index2 = i;
            } else if (over3) {
                top3 = a; bits3 = a_bits;
            }
        }
        uint32_t scale_raw;
        if (topk == 0) scale_raw = bits1;
        else if (topk == 1) {
            if (index1 < 0) { index1 = 0; scale_raw = wide ? raw[1] : (raw[1] & sign_clear); }
            else scale_raw = bits2;
        } else {
            if (index1 < 0) { index1 = 0; index2 = 1; scale_raw = 0; }
            else if (index2 < 0) { index2 = (index1 + 1) % g; scale_raw = 0; }
            else scale_raw = bits3;
        }
        const uint32_t top1_raw = topk >= 1 ? raw[index1] : 0, top2_raw = topk == 2 ? raw[index2] : 0;
        if (topk >= 1) v[index1] = 0.0f;
        if (topk == 2) v[index2] = 0.0f;

        /* encode in scan order (the order fixes which uniform an element receives) */
        float scale = raw_to_f32(scale_raw, dtype);
        if (scale < 1e-6) scale = 1e-6f;
        const float levels = bit == 8 ? 127.0f : 7.0f;
        const float multiplier = (float)((double)levels / (double)scale);
        philox_state stream;
        if (stochastic) stream_init(&stream, seed, (uint64_t)group, offset);
        int code[256];
        for (int j = 0; j < g; ++j) {
            const int i = (start + j) & (g - 1);
            if (kind == 0) {
                float t;
                if (stochastic) {
                    const float noise = (float)((double)stream_uniform(&stream) - 0.5);
                    t = fmaf(v[i], multiplier, noise);
                } else t = v[i] * multiplier;
                const float r = rintf(t);
                code[i] = r != r ? 0 : (r > levels ? (int)levels : (r < -levels ? -(int)levels : (int)r));
            } else {
                const float *book = BOOKS[kind - 1];
                const float t = v[i] / scale;
                int lo = 0, hi = 14;
                while (lo < hi) {
                    const int mid = (lo + hi + 1) / 2;
                    if (t < book[mid]) hi = mid - 1; else lo = mid;
                }
                if (stochastic) {
                    const float q = stream_uniform(&stream);
                    if (q < (t - book[lo]) / (book[lo + 1] - book[lo])) ++lo;
                } else if (t - book[lo] > (book[lo + 1] - book[lo]) / 2) ++lo;
                code[i] = lo;
            }
        }

        /* pack: the first code of a word of `item` bytes sits in its most significant byte / nibble */
        uint8_t *codes = payload + codes_at(group, cb, mb, compact);
        const int per_word = item * 8 / bit;
        for (int w = 0; w < g / per_word; ++w) {
            uint32_t word = 0;
            for (int k = 0; k < per_word; ++k)
                word = (word << bit) | ((uint32_t)code[w * per_word + k] & (bit == 8 ? 0xFFu : 0xFu));
            put_word(codes + w * item, word, item);
        }
        uint8_t *meta = payload + meta_at(group, groups, cb, mb, compact);
        put_word(meta, scale_raw, item);
        if (topk == 1) {
            put_word(meta + item, (uint32_t)index1, item);
            put_word(meta + 2 * item, top1_raw, item);
        } else if (topk == 2) {
            put_word(meta + item, (uint32_t)(index1 | (index2 << 8)), item);
            put_word(meta + 2 * item, top1_raw, item);
            put_word(meta + 3 * item, top2_raw, item);
        }
    }
}

/* ---- dequantize ---------------------------------------------------------------------------- */
static float add_once(float a, float b, int dtype) {   /* a + b rounded once to dtype */
    if (dtype == G_F32) return a + b;
    const double wide = (double)a + (double)b;
    float near = (float)wide;
    const double err = wide - (double)near;
    if (err != 0.0 && isfinite(near)) {
        uint32_t u = f32_to_bits(near);
        if ((u & 1u) == 0) {
            u = ((err > 0.0) == (near > 0.0f)) ? u + 1u : u - 1u;
            near = bits_to_f32(u);
        }
    }
    return raw_to_f32(f32_to_raw(near, dtype), dtype);
}

/* op: 0 none, 1 sum, 2 max, 3 min; out is read for op != 0 */
void lbg_dequantize(const uint8_t *payload, int64_t numel, int g, int bit, int kind, int topk, int compact, int dtype,
                    int op, void *out) {
    const int item = item_of(dtype);
    const int cb = g * bit / 8, mb = meta_words(topk) * item;
    const int64_t groups = numel / g;
    const int per_word = item * 8 / bit;
    uint32_t result[256];
    for (int64_t group = 0; group < groups; ++group) {
        const uint8_t *codes = payload + codes_at(group, cb, mb, compact);
        const uint8_t *meta = payload + meta_at(group, groups, cb, mb, compact);
        const float scale = raw_to_f32(get_word(meta, item), dtype);
        const float step = kind == 0 ? (float)((double)scale / (bit == 8 ? 127.0 : 7.0)) : scale;
        for (int i = 0; i < g; ++i) {
            const uint32_t word = get_word(codes + (i / per_word) * item, item);
            const int shift = bit * (per_word - 1 - i % per_word);
            const uint32_t field = (word >> shift) & (bit == 8 ? 0xFFu : 0xFu);
            float value;
            if (kind != 0) value = BOOKS[kind - 1][field] * step;
            else if (bit == 8) value = (float)(int8_t)field * step;
            else value = (float)(field >= 8 ? (int)field - 16 : (int)field) * step;
            result[i] = f32_to_raw(value, dtype);
        }
        if (topk >= 1) {
            const uint32_t indices = get_word(meta + item, item);
            result[indices & 0xFFu] = get_word(meta + 2 * item, item);
            if (topk == 2) result[(indices >> 8) & 0xFFu] = get_word(meta + 3 * item, item);
        }
        for (int i = 0; i < g; ++i) {
            const int64_t e = group * g + i;
            uint32_t raw = result[i];
            if (op != 0) {
                const uint32_t old_raw = raw_at(out, e, dtype);
                const float old = raw_to_f32(old_raw, dtype), v = raw_to_f32(raw, dtype);
                if (op == 1) raw = f32_to_raw(add_once(old, v, dtype), dtype);
                else if (op == 2) raw = old > v ? old_raw : raw;
                else raw = old > v ? raw : old_raw;
            }
            put_word((uint8_t *)out + e * item, raw, item);
        }
    }
}
