// Exhaustive check of the division-free scale formula used by the HIP quantizer:
// for every non-negative finite float a,
//   q0 = a*c; r = fma(-q0,127,a); q1 = fma(r,c,q0)   with c = RN(1/127) = 0x3C010204
// must equal the correctly rounded a/127 (what the reference's torch division yields).
// Exit status 0 = no mismatch.  Build: gcc -O2 -mfma -fopenmp -ffp-contract=off check_scale127.c -lm
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <omp.h>
int main(void) {
    const float c = 1.0f / 127.0f;
    uint32_t cb; memcpy(&cb, &c, 4);
    printf("c bits = 0x%08X\n", cb);
    long long bad = 0, bad_small = 0;
    #pragma omp parallel for reduction(+:bad,bad_small) schedule(static)
    for (uint64_t b = 0; b < 0x7F800000ull; ++b) {
        uint32_t bits = (uint32_t)b; float a; memcpy(&a, &bits, 4);
        float want = a / 127.0f;
        float q0 = a * c;
        float r = fmaf(-q0, 127.0f, a);
        float q1 = fmaf(r, c, q0);
        if (q1 != want) { if (want >= 5.9604645e-08f) bad++; else bad_small++; }
    }
    printf("mismatches with result >= 2^-24: %lld ; below (clamped region): %lld\n", bad, bad_small);
    return bad != 0;
}
