// Exhaustive check that adding two fp16 (or two bfloat16) values in fp32 and rounding the fp32 sum to the
// 16-bit type gives the correctly rounded sum of the two values, i.e. what a native 16-bit add returns.
// The kernels of the CUDA byte format rely on it for their SUM combine: both operands are values of the 16-bit
// type, the sum is formed by one fp32 add and converted once.  (fp32 carries 24 significand bits, at least
// 2p + 2 for p = 11 and p = 8, which is the known condition for the second rounding to be harmless; this program
// does not take that on trust.)
//
// For every ordered pair of finite values: the exact sum is formed in double (exact when the exponents are at
// most 40 apart; beyond that the smaller operand cannot move the result off the larger one, which is checked
// as such), rounded once to the type, and compared with the fp32 sum rounded to the type.
// Exit status 0 = no mismatch.  Build: gcc -O2 -fopenmp -ffp-contract=off check_half_sum.c -lm
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef struct { int p, emin, emax; } format;   // significand bits, smallest and largest normal exponent
static const format HALF = {11, -14, 15}, BFLOAT = {8, -126, 127};

static double value_of(uint32_t bits, format f) {   // finite values only
    const int ebits = 16 - f.p, bias = f.emax;
    const uint32_t sign = bits >> 15, e = (bits >> (f.p - 1)) & ((1u << ebits) - 1), m = bits & ((1u << (f.p - 1)) - 1);
    const double mag = e == 0 ? ldexp((double)m, f.emin - (f.p - 1)) : ldexp((double)(m | (1u << (f.p - 1))), (int)e - bias - (f.p - 1));
    return sign ? -mag : mag;
}

// x rounded to nearest even in the format; x is exact in double and the scaling is by a power of two.
static double round_to(double x, format f) {
    if (x == 0.0) return x;
    int e;
    frexp(x, &e);                       // |x| in [2^(e-1), 2^e)
    int ulp_exp = (e - 1 < f.emin ? f.emin : e - 1) - (f.p - 1);
    double r = ldexp(nearbyint(ldexp(x, -ulp_exp)), ulp_exp);
    const double limit = ldexp(1.0, f.emax + 1);
    if (fabs(r) >= limit) r = x > 0 ? INFINITY : -INFINITY;
    return r;
}

static long long check(format f, const char *name) {
    const int ebits = 16 - f.p;
    const uint32_t exp_all_ones = ((1u << ebits) - 1) << (f.p - 1);
    long long bad = 0, pairs = 0;
    #pragma omp parallel for reduction(+:bad,pairs) schedule(dynamic, 64)
    for (uint32_t ia = 0; ia < 65536; ++ia) {
        if ((ia & exp_all_ones) == exp_all_ones) continue;          // infinities and NaNs
        const double a = value_of(ia, f);
        for (uint32_t ib = 0; ib <= ia; ++ib) {
            if ((ib & exp_all_ones) == exp_all_ones) continue;
            const double b = value_of(ib, f);
            const float sum32 = (float)a + (float)b;                // one IEEE fp32 add
            const double through_float = isinf(sum32) ? (double)sum32 : round_to((double)sum32, f);
            double once;
            int ea, eb;
            frexp(a, &ea); frexp(b, &eb);
            if (a != 0.0 && b != 0.0 && abs(ea - eb) > 40) once = fabs(a) > fabs(b) ? a : b;
            else once = round_to(a + b, f);                         // a + b is exact here
            ++pairs;
            if (!(once == through_float) || signbit(once) != signbit(through_float)) ++bad;
        }
    }
    printf("%s: %lld pairs, %lld mismatches\n", name, pairs, bad);
    return bad;
}

int main(void) {
    long long bad = check(HALF, "fp16") + check(BFLOAT, "bfloat16");
    return bad != 0;
}
