/*
 * Scalar C restatement of the INT8 group codec.  TEST INFRASTRUCTURE ONLY.
 *
 * One element at a time, no vector intrinsics, compiled with
 * -ffp-contract=off so that every product and sum is rounded separately.
 * It exists to pin the numpy and torch restatements from a third, independent
 * direction; the product never links it.
 *
 * Reference lines followed (paths under the upstream repository):
 *   lbo_quantize_f32      ccdl_comm/quantization/torch_fallback.py:24-36,56-61
 *   lbo_dequantize_f32    ccdl_comm/quantization/torch_fallback.py:48-53
 *   lbo_reduce_f32        ccdl_comm/communication/gather_reduce.py:27-45
 *   lbo_ef_step_*         ccdl_comm/quantization/error_feedback.py:27-41,
 *                         ccdl_comm/communication/ddp.py:69-97
 *
 * Undefined-by-reference values: a NaN quotient encodes as 0, an infinite one
 * saturates to +-127; the scale keeps its NaN/Inf bits.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define LBO_EPS 1.1920928955078125e-07f /* 2^-23 */

static float bf16_bits_to_f32(uint16_t bits) {
    uint32_t u = (uint32_t)bits << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t f32_to_bf16_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static int8_t encode_one(float x, float scale) {
    float q = rintf(x / scale); /* default rounding mode: nearest-even */
    if (q != q) return 0;
    if (q > 127.0f) return 127;
    if (q < -127.0f) return -127;
    return (int8_t)q;
}

static float group_scale(const float *x, int64_t count) {
    float absmax = 0.0f;
    int saw_nan = 0;
    for (int64_t i = 0; i < count; ++i) {
        float a = fabsf(x[i]);
        if (a != a) saw_nan = 1;
        if (a > absmax) absmax = a;
    }
    if (saw_nan) return NAN;
    float s = absmax / 127.0f;
    return s < LBO_EPS ? LBO_EPS : s;
}

/* codes must hold ceil(n/g)*g bytes, scales ceil(n/g) floats. */
void lbo_quantize_f32(const float *x, int64_t n, int group_size, int8_t *codes, float *scales) {
    int64_t groups = (n + group_size - 1) / group_size;
    for (int64_t g = 0; g < groups; ++g) {
        int64_t base = g * group_size;
        int64_t live = n - base < group_size ? n - base : group_size;
        float s = group_scale(x + base, live);
        scales[g] = s;
        for (int64_t i = 0; i < group_size; ++i)
            codes[base + i] = i < live ? encode_one(x[base + i], s) : 0;
    }
}

void lbo_dequantize_f32(const int8_t *codes, const float *scales, int64_t n, int group_size, float *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = (float)codes[i] * scales[i / group_size];
}

/* Left fold in payload order; divisor > 1 applies a true division at the end. */
void lbo_reduce_f32(const int8_t *const *codes, const float *const *scales, int world, int64_t n,
                    int group_size, float divisor, float *out) {
    for (int64_t i = 0; i < n; ++i) {
        float total = (float)codes[0][i] * scales[0][i / group_size];
        for (int r = 1; r < world; ++r) {
            float term = (float)codes[r][i] * scales[r][i / group_size];
            total = total + term;
        }
        out[i] = divisor == 1.0f ? total : total / divisor;
    }
}

/*
 * One error-feedback bucket step on a bf16 gradient with an fp32 residual:
 *   p = float(g) + r;  q = quant(p);  restored = code*scale (optionally rounded
 *   to bf16);  r' = p - restored.
 * residual_in may be NULL (no residual yet).  restored_bf16 != 0 rounds the
 * decoded value to bf16 before the subtraction and writes bf16 bits to
 * restored_out (uint16), else restored_out receives float.
 */
void lbo_ef_step_bf16(const uint16_t *grad_bits, const float *residual_in, int64_t n, int group_size,
                      int8_t *codes, float *scales, float *residual_out, void *restored_out,
                      int restored_bf16) {
    int64_t groups = (n + group_size - 1) / group_size;
    float p[64];
    for (int64_t g = 0; g < groups; ++g) {
        int64_t base = g * group_size;
        int64_t live = n - base < group_size ? n - base : group_size;
        for (int64_t i = 0; i < live; ++i) {
            float v = bf16_bits_to_f32(grad_bits[base + i]);
            p[i] = residual_in ? v + residual_in[base + i] : v;
        }
        float s = group_scale(p, live);
        scales[g] = s;
        for (int64_t i = 0; i < group_size; ++i) {
            if (i >= live) { codes[base + i] = 0; continue; }
            int8_t c = encode_one(p[i], s);
            codes[base + i] = c;
            float restored = (float)c * s;
            if (restored_bf16) {
                uint16_t bits = f32_to_bf16_bits(restored);
                if (restored_out) ((uint16_t *)restored_out)[base + i] = bits;
                restored = bf16_bits_to_f32(bits);
            } else if (restored_out) {
                ((float *)restored_out)[base + i] = restored;
            }
            residual_out[base + i] = p[i] - restored;
        }
    }
}

/* Same step for an fp32 gradient. */
void lbo_ef_step_f32(const float *grad, const float *residual_in, int64_t n, int group_size,
                     int8_t *codes, float *scales, float *residual_out, float *restored_out) {
    int64_t groups = (n + group_size - 1) / group_size;
    float p[64];
    for (int64_t g = 0; g < groups; ++g) {
        int64_t base = g * group_size;
        int64_t live = n - base < group_size ? n - base : group_size;
        for (int64_t i = 0; i < live; ++i)
            p[i] = residual_in ? grad[base + i] + residual_in[base + i] : grad[base + i];
        float s = group_scale(p, live);
        scales[g] = s;
        for (int64_t i = 0; i < group_size; ++i) {
            if (i >= live) { codes[base + i] = 0; continue; }
            int8_t c = encode_one(p[i], s);
            codes[base + i] = c;
            float restored = (float)c * s;
            if (restored_out) restored_out[base + i] = restored;
            residual_out[base + i] = p[i] - restored;
        }
    }
}
