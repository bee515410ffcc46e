// Evidence for the quantizer's division-free exact quotient (csrc/device_utils.h: encode_group): for dividends p
// and scales s from its domain (|p| <= 127.5 s, s >= 2^-23), q1 = fma(fma(-q0, s, p), y, q0) with y = 1/s and
// q0 = p*y is compared on the device with the division p/s, bit for bit, and so are the codes rint() makes of
// them.  Modes: 0 random, 1 scale mantissa (almost) all ones, 2 scales with few mantissa bits, 3 and 4 dividends
// within four ulps of (k + 0.5) * s, 5 dividends with 8 or 11 significant bits (bf16 / fp16 tensors).
// Usage: quotient_check [rounds per mode, 4.3e9 pairs each].  Exit status 1 when a code differs; quotients that
// differ only for denormal dividends (a remainder that underflows) are reported and do not fail the check.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
__device__ __forceinline__ uint32_t mix(uint64_t x) { x ^= x >> 33; x *= 0xff51afd7ed558ccdULL; x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ULL; x ^= x >> 33; return (uint32_t)x; }
__global__ void check(uint64_t seed, int mode, unsigned long long *bad, unsigned long long *bad_code, float *ex) {
    uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    unsigned long long nb = 0, nc = 0;
    for (int it = 0; it < 4096; ++it) {
        uint64_t h = seed * 0x9E3779B97F4A7C15ULL + id * 4096 + it;
        uint32_t a = mix(h), b = mix(h ^ 0xDEADBEEFCAFEULL), c = mix(h + 0x1234567ULL);
        // scale: random normal float with exponent in [-23+127 .. 20+127]
        uint32_t sexp = 104 + (a % 44);
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
        const float y = 1.0f / s;
        const float q0 = p * y;
        const float rem = __builtin_fmaf(-q0, s, p);
        const float q1 = __builtin_fmaf(rem, y, q0);
        const float want = p / s;
        if (__float_as_uint(q1) != __float_as_uint(want)) { ++nb; ex[0] = p; ex[1] = s; }
        if (__builtin_rintf(q1) != __builtin_rintf(want)) ++nc;
    }
    if (nb) atomicAdd(bad, nb);
    if (nc) atomicAdd(bad_code, nc);
}
int main(int argc, char **argv) {
    int rounds = argc > 1 ? atoi(argv[1]) : 8;
    unsigned long long *bad, *bad_code; float *ex;
    if (hipMalloc(&bad, 8) != hipSuccess || hipMalloc(&bad_code, 8) != hipSuccess || hipMalloc(&ex, 8) != hipSuccess) return 2;
    unsigned long long total = 0;
    for (int mode = 0; mode <= 5; ++mode) {
        if (hipMemset(bad, 0, 8) != hipSuccess || hipMemset(bad_code, 0, 8) != hipSuccess) return 2;
        for (int r = 0; r < rounds; ++r) hipLaunchKernelGGL(check, dim3(4096), dim3(256), 0, 0, (uint64_t)(mode * 1000 + r + 1), mode, bad, bad_code, ex);
        unsigned long long hb, hc; float he[2];
        if (hipMemcpy(&hb, bad, 8, hipMemcpyDeviceToHost) != hipSuccess || hipMemcpy(&hc, bad_code, 8, hipMemcpyDeviceToHost) != hipSuccess ||
            hipMemcpy(he, ex, 8, hipMemcpyDeviceToHost) != hipSuccess) return 2;
        unsigned long long n = (unsigned long long)rounds * 4096ULL * 256ULL * 4096ULL;
        printf("mode %d: %llu pairs, quotient mismatches %llu, code mismatches %llu (example p=%a s=%a)\n", mode, n, hb, hc, he[0], he[1]);
        total += hc;
    }
    printf("CODE MISMATCHES %llu\n", total);
    return total ? 1 : 0;
}
