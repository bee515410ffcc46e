/*
 * fp16 / bf16 <-> float conversions shared by the scalar C restatements.  TEST INFRASTRUCTURE ONLY.
 * Hand-written bit manipulation (round to nearest, ties to even) so that nothing is shared with numpy.
 */
#ifndef ORACLE_SCALAR_FLOATS_H
#define ORACLE_SCALAR_FLOATS_H
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0x1Fu) return bits_to_f32(sign | 0x7F800000u | (man << 13));
    if (exp == 0) {
        float v = (float)man * 0x1p-24f; /* subnormal: man * 2^-24, exact */
        return sign ? -v : v;
    }
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline uint16_t f32_to_f16(float f) { /* round to nearest, ties to even */
    uint32_t u = f32_to_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x3FFu));
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);          /* >= 65536 (incl. inf) */
    if (a < 0x38800000u) {                                            /* below the smallest normal half */
        float scaled = fabsf(f) * 0x1p24f;                            /* exact scaling; < 1024 */
        float r = rintf(scaled);                                      /* nearest-even in units of 2^-24 */
        return (uint16_t)(sign | (uint16_t)r);                        /* r == 1024 lands on the first normal */
    }
    uint32_t lsb = (a >> 13) & 1u;
    a += 0xFFFu + lsb;
    uint32_t h = (a >> 13) - (112u << 10);
    if (h >= 0x7C00u) h = 0x7C00u;                                    /* rounded up to infinity */
    return (uint16_t)(sign | h);
}

#endif
