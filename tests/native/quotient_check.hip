// Evidence for the quantizer's division-free exact quotient (csrc/device_utils.h: encode_group): for dividends p
// and scales s from its domain (|p| <= 127.5 s, 2^-23 <= s <= FLT_MAX / 127), q1 = fma(fma(-q0, s, p), y, q0) with
// y = 1/s and q0 = p*y is compared on the device with the division p/s, bit for bit, and so are the codes rint()
// makes of them.
//
// Sampled modes, scale exponents over the whole domain (2^-23 .. 2^120): 0 random, 1 scale mantissa (almost) all
// ones, 2 scales with few mantissa bits, 3 and 4 dividends within four ulps of (k + 0.5) * s, 5 dividends with 8 or
// 11 significant bits (bf16 / fp16 tensors).
//
// Exhaustive mode 6.  q1 and the correctly rounded quotient are equal or neighbouring floats, and every half-integer
// up to 127.5 is a float, so the two can round to different codes only when one of them IS a half-integer, i.e. when
// p lies within a few ulps of (k + 0.5) * s.  The operations are invariant under multiplying s and p by a power of
// two as long as nothing underflows or overflows, which cannot happen for |p/s| >= 0.5 in the domain.  So mode 6
// walks every one of the 2^23 mantissas of s (at exponent 0, and again at both ends of the exponent range), all 256
// half-integers k + 0.5 in (-128, 128) and the 13 dividends within six ulps of RN((k + 0.5) * s): every case in
// which the refined quotient could change a code.
//
// Mode 7 is the other division-free quotient of the library (csrc/cuda_wire_general.hip, code-book quantizer):
// the compiler's own expansion of v / s - v_rcp_f32, a Newton step, product, two corrections - with the reciprocal
// part shared by the elements that have the same divisor and without the operand scaling and fix-up instructions,
// for divisors in [2^-60, 2^60] and |v| <= s.  It must equal v / s bit for bit for every quotient of 2^-40 and
// above.  Below that the caller does not look at the bits: such a quotient lies between the code book's zero and
// its neighbours by less than their rounding error, so it encodes as the zero entry whatever its last bits are -
// and that is where the two forms do differ, for dividends so small (below 2^-103) that the hardware division
// rescales them first.  Sampled over random divisors and dividends of every magnitude down to the denormals,
// 4.3e9 pairs a round.
//
// Usage: quotient_check [rounds per sampled mode, 4.3e9 pairs each; 0 skips them] [exhaustive 0|1, default 1].
// Exit status 1 when a code differs or a quotient differs for |p/s| >= 2^-64; below that the exact remainder
// fma(-q0, s, p) can underflow and lose its last bits, the code is 0 either way, and such pairs are only counted.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
__device__ __forceinline__ uint32_t mix(uint64_t x) { x ^= x >> 33; x *= 0xff51afd7ed558ccdULL; x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ULL; x ^= x >> 33; return (uint32_t)x; }
struct Tally { unsigned long long tiny, quotient, code; };
__device__ __forceinline__ void compare(float p, float s, Tally &t, float *ex) {
    const float y = 1.0f / s;
    const float q0 = p * y;
    const float rem = __builtin_fmaf(-q0, s, p);
    const float q1 = __builtin_fmaf(rem, y, q0);
    const float want = p / s;
    if (__float_as_uint(q1) != __float_as_uint(want)) {
        if (fabsf(want) < 0x1p-64f) ++t.tiny; else { ++t.quotient; ex[0] = p; ex[1] = s; }
    }
    if (__builtin_rintf(q1) != __builtin_rintf(want)) { ++t.code; ex[0] = p; ex[1] = s; }
}
__device__ __forceinline__ void publish(const Tally &t, unsigned long long *bad) {
    if (t.tiny) atomicAdd(bad, t.tiny);
    if (t.quotient) atomicAdd(bad + 1, t.quotient);
    if (t.code) atomicAdd(bad + 2, t.code);
}
// One lane per scale mantissa; `sexp` is the biased exponent of every scale of the launch.
__global__ void check_all_ties(uint32_t sexp, unsigned long long *bad, float *ex) {
    const uint32_t sman = blockIdx.x * blockDim.x + threadIdx.x;
    const float s = __uint_as_float((sexp << 23) | sman);
    Tally t = {0, 0, 0};
    for (int k = -128; k <= 127; ++k) {
        const float base = ((float)k + 0.5f) * s;
        for (int ulps = -6; ulps <= 6; ++ulps) {
            const float p = __uint_as_float(__float_as_uint(base) + ulps);
            if (fabsf(p) <= 127.5f * s) compare(p, s, t, ex);
        }
    }
    publish(t, bad);
}
__global__ void check_shared_reciprocal(uint64_t seed, unsigned long long *bad, float *ex) {
    uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    Tally t = {0, 0, 0};
    for (int it = 0; it < 1024; ++it) {
        uint64_t h = seed * 0x9E3779B97F4A7C15ULL + id * 1024 + it;
        uint32_t a = mix(h), b = mix(h ^ 0xDEADBEEFCAFEULL);
        const float s = __uint_as_float(((67u + a % 121u) << 23) | (b & 0x7FFFFF));      // 2^-60 .. 2^60
        float r = __builtin_amdgcn_rcpf(s);
        r = __builtin_fmaf(__builtin_fmaf(-s, r, 1.0f), r, r);
        for (int e = 0; e < 4; ++e) {                                                    // four dividends a divisor
            uint32_t c = mix(h + 0x1234567ULL * (e + 1));
            float v;
            if (e == 0) v = s * (((float)(c & 0xFFFFFF) / 16777216.0f) * 2.0f - 1.0f);   // anywhere in [-s, s]
            else if (e == 1) v = __uint_as_float(__float_as_uint(s) - (c & 0xFFFF));      // just below s
            else if (e == 2) v = __uint_as_float(c & 0x7FFFFFFF);                         // any exponent
            else v = __uint_as_float((__float_as_uint(s) & 0x7F800000u) - ((c % 90) << 23) | (c & 0x7FFFFF)); // scaled down
            if (!(fabsf(v) <= s)) continue;
            float q = v * r;
            q = __builtin_fmaf(__builtin_fmaf(-s, q, v), r, q);
            q = __builtin_fmaf(__builtin_fmaf(-s, q, v), r, q);
            const float want = v / s;
            if (__float_as_uint(q) != __float_as_uint(want)) {
                if (fabsf(want) < 0x1p-40f) ++t.tiny; else { ++t.quotient; ex[0] = v; ex[1] = s; }
            }
        }
    }
    publish(t, bad);
}
__global__ void check(uint64_t seed, int mode, unsigned long long *bad, float *ex) {
    uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    Tally t = {0, 0, 0};
    for (int it = 0; it < 4096; ++it) {
        uint64_t h = seed * 0x9E3779B97F4A7C15ULL + id * 4096 + it;
        uint32_t a = mix(h), b = mix(h ^ 0xDEADBEEFCAFEULL), c = mix(h + 0x1234567ULL);
        // scale: random normal float with exponent in [-23+127 .. 120+127]: eps up to FLT_MAX / 127
        uint32_t sexp = 104 + (a % 144);
        uint32_t sman = b & 0x7FFFFF;
        if (mode == 1) sman = 0x7FFFFF - (b & 7);                 // mantissa (almost) all ones
        if (mode == 2) sman &= 0x7F0000;                           // few mantissa bits (bf16-like scale sources)
        float s = __uint_as_float((sexp << 23) | sman);
        float p;
        if (mode == 3 || mode == 4) {                              // p next to (k + 0.5) * s
            float k = (float)((int)(c % 255) - 127);
            float base = (k + 0.5f) * s;
            int ulps = (int)((c >> 8) % 9) - 4;
            p = __uint_as_float(__float_as_uint(base) + ulps);
        } else if (mode == 5) {                                    // bf16 / fp16 like p: few mantissa bits
            float q = ((float)(c & 0xFFFFFF) / 16777216.0f) * 254.0f - 127.0f;
            p = q * s;
            uint32_t bits = __float_as_uint(p);
            bits &= (c & 1) ? 0xFFFF0000u : 0xFFFFE000u;
            p = __uint_as_float(bits);
        } else {
            float q = ((float)(c & 0xFFFFFF) / 16777216.0f) * 254.0f - 127.0f;
            p = q * s;
            p = __uint_as_float(__float_as_uint(p) ^ ((c >> 24) & 3));
        }
        if (!(fabsf(p) <= 127.5f * s)) continue;
        compare(p, s, t, ex);
    }
    publish(t, bad);
}
int main(int argc, char **argv) {
    const int rounds = argc > 1 ? atoi(argv[1]) : 8;
    const int exhaustive = argc > 2 ? atoi(argv[2]) : 1;
    unsigned long long *bad; float *ex;
    if (hipMalloc(&bad, 24) != hipSuccess || hipMalloc(&ex, 8) != hipSuccess) return 2;
    unsigned long long failures = 0;
    for (int mode = 0; mode <= 7; ++mode) {
        if (mode == 6 ? !exhaustive : rounds == 0) continue;
        if (hipMemset(bad, 0, 24) != hipSuccess || hipMemset(ex, 0, 8) != hipSuccess) return 2;
        unsigned long long n;
        if (mode < 6) {
            for (int r = 0; r < rounds; ++r) hipLaunchKernelGGL(check, dim3(4096), dim3(256), 0, 0, (uint64_t)(mode * 1000 + r + 1), mode, bad, ex);
            n = (unsigned long long)rounds * 4096ULL * 256ULL * 4096ULL;
        } else if (mode == 7) {
            for (int r = 0; r < rounds; ++r) hipLaunchKernelGGL(check_shared_reciprocal, dim3(4096), dim3(256), 0, 0, (uint64_t)(7000 + r), bad, ex);
            n = (unsigned long long)rounds * 4096ULL * 256ULL * 4096ULL;
        } else {
            const uint32_t exponents[3] = {127, 104, 247};      // 1, the smallest scale, the largest the domain holds
            for (uint32_t sexp : exponents) hipLaunchKernelGGL(check_all_ties, dim3((1u << 23) / 256), dim3(256), 0, 0, sexp, bad, ex);
            n = 3ULL * (1ULL << 23) * 256ULL * 13ULL;
        }
        unsigned long long h[3]; float he[2];
        if (hipDeviceSynchronize() != hipSuccess || hipMemcpy(h, bad, 24, hipMemcpyDeviceToHost) != hipSuccess ||
            hipMemcpy(he, ex, 8, hipMemcpyDeviceToHost) != hipSuccess) return 2;
        printf("mode %d: %llu pairs, quotient mismatches %llu (and %llu too small to matter), code mismatches %llu (example p=%a s=%a)\n",
               mode, n, h[1], h[0], h[2], he[0], he[1]);
        failures += h[1] + h[2];
    }
    printf("MISMATCHES %llu\n", failures);
    return failures ? 1 : 0;
}
