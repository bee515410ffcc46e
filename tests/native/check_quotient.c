// CPU check of the quantizer's division-free quotient (csrc/device_utils.h: encode_group) on the cases that decide
// a code: y = 1/s (IEEE), q0 = p*y, q1 = fma(fma(-q0, s, p), y, q0) against p/s, for
//   every scale with at most 11 significant mantissa bits (what a group of fp16 / bf16 values, or of fp32 values
//     from a short computation, produces as absmax/127 candidates) and the all-ones and near-all-ones mantissas,
//     at the smallest, a middle and the largest exponent of the scale's domain, plus 2^22 random mantissas, and
//   every dividend within 8 ulps of (k + 0.5) * s for k = -128 .. 127 (the rounding ties) and of k * s.
// rint(q1) must equal rint(p/s) always, and q1 must equal p/s bit for bit.  The device test
// (tests/native/quotient_check.hip) walks all 2^23 mantissas on the GPU; this one needs no GPU.
// Exit status 0 = no mismatch.  Build: gcc -O2 -mfma -fopenmp -ffp-contract=off check_quotient.c -lm
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <omp.h>
static float from_bits(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
static uint32_t to_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }
static uint32_t mix(uint64_t x) { x ^= x >> 33; x *= 0xff51afd7ed558ccdULL; x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ULL; x ^= x >> 33; return (uint32_t)x; }
int main(void) {
    const uint32_t exponents[3] = {104, 127, 247};          // 2^-23 (the smallest scale), 1, 2^120
    const int structured = 1 << 12, random = 1 << 22;       // 11 explicit bits + the all-ones family; random mantissas
    long long pairs = 0, bad_code = 0, bad_quotient = 0;
    #pragma omp parallel for reduction(+:pairs,bad_code,bad_quotient) schedule(dynamic, 4096)
    for (int64_t m = 0; m < structured + random; ++m) {
        uint32_t mantissa;
        if (m < (1 << 11)) mantissa = (uint32_t)m << 12;                        // 11 leading bits, zeros behind
        else if (m < structured) mantissa = 0x7FFFFFu - (uint32_t)(m - (1 << 11));   // all ones and just below
        else mantissa = mix((uint64_t)m * 0x9E3779B97F4A7C15ULL) & 0x7FFFFFu;
        for (int e = 0; e < 3; ++e) {
            if (m >= structured && e != 1) continue;                            // random mantissas at one exponent
            const float s = from_bits((exponents[e] << 23) | mantissa);
            const float y = 1.0f / s;
            for (int twice_k = -256; twice_k <= 255; ++twice_k) {               // k*s and (k + 0.5)*s
                const float base = (0.5f * (float)twice_k) * s;
                for (int ulps = -8; ulps <= 8; ++ulps) {
                    const float p = from_bits(to_bits(base) + (uint32_t)ulps);
                    if (!(fabsf(p) <= 127.5f * s)) continue;
                    const float q0 = p * y;
                    const float q1 = fmaf(fmaf(-q0, s, p), y, q0);
                    const float want = p / s;
                    ++pairs;
                    if (rintf(q1) != rintf(want)) ++bad_code;
                    if (to_bits(q1) != to_bits(want) && fabsf(want) >= 0x1p-64f) ++bad_quotient;
                }
            }
        }
    }
    printf("pairs %lld, code mismatches %lld, quotient mismatches %lld\n", pairs, bad_code, bad_quotient);
    return bad_code != 0 || bad_quotient != 0;
}
