// Device-side helpers shared by the gfx950 codec kernels: 16-bit float types,
// vector load/store, wavefront-row (DPP) reductions and the exact arithmetic
// primitives the wire format depends on.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lbc {

using f16 = _Float16;
using bf16 = __bf16;

#ifndef LBC_BLOCK
#define LBC_BLOCK 256
#endif
#ifndef LBC_TILE_ORDER
#define LBC_TILE_ORDER 0
#endif
constexpr int kWave = 64;
constexpr int kBlock = LBC_BLOCK;
constexpr int kWavesPerBlock = kBlock / kWave;

// Index of the u-th tile a wavefront handles inside its block.  Order 0: the block's
// wavefronts sweep the block's span together (tile = u * waves + wave); order 1: each
// wavefront owns UNROLL consecutive tiles.
template <int UNROLL> __device__ __forceinline__ int tile_in_block(int u, int wave) {
    return LBC_TILE_ORDER == 0 ? u * kWavesPerBlock + wave : wave * UNROLL + u;
}
// Workgroups of a grid are dealt round-robin to the chip's 8 XCDs.  When the x range of a launch covers at most
// LBC_XCD_SPAN_ELEMS elements (shard-sized reduces, per-chunk rows of the chunked quantize: an eighth of the range
// is then no more than a 2 MiB page of the widest tensor), letting every XCD walk one contiguous eighth measured
// up to 7 % faster and never slower; for larger ranges the round-robin order, which keeps all XCDs on one moving front of addresses and
// pages, measured 5-12 % faster, so those keep it.  The remainder of a grid that is not a multiple of 8 keeps its
// place.
#ifndef LBC_XCD_SPAN_ELEMS
#define LBC_XCD_SPAN_ELEMS (1 << 22)
#endif
template <bool ALWAYS = false>
__device__ __forceinline__ unsigned xcd_contiguous_block(unsigned block, unsigned grid, int block_elems) {
    const unsigned per_xcd = grid >> 3;
    const bool in_span = ALWAYS || static_cast<int64_t>(grid) * block_elems <= LBC_XCD_SPAN_ELEMS;
    const bool remap = in_span && block < (per_xcd << 3);
    return remap ? (block & 7u) * per_xcd + (block >> 3) : block;
}
template <bool ALWAYS = false>
__device__ __forceinline__ unsigned xcd_contiguous_block(int block_elems) {
    return xcd_contiguous_block<ALWAYS>(blockIdx.x, gridDim.x, block_elems);
}
constexpr uint32_t kEpsBits = 0x34000000u;  // 2^-23, torch.finfo(float32).eps

// Access modes of the bulk loads and stores.  kScalar: element by element (any
// alignment).  kVector: one vector instruction per lane (the caller guarantees
// N*sizeof(T) alignment), plain cached accesses - for operands that are known to
// sit in the last-level cache.  kStream: vector instructions with the
// non-temporal hint on the loads - every tensor here is read once, and when it is
// not already cached the hint measured 10-25 % more bandwidth at every size from
// 16 MB to 600 MB of traffic (with it the time no longer depends on what the
// 256 MiB memory-side cache holds; cached loads are ~5 % faster only when
// everything is resident).  Stores under kStream are chosen per kernel.
// kStreamThrough (fused reduce only): kStream with write-through stores.
enum AccessMode { kScalar = 0, kVector = 1, kStream = 2, kStreamThrough = 3 };

template <typename T, int N>
using vec_t = T __attribute__((ext_vector_type(N)));

template <typename T> struct is_void_t { static constexpr bool value = false; };
template <> struct is_void_t<void> { static constexpr bool value = true; };

template <bool PICK_FIRST, typename A, typename B> struct pick_t { using type = A; };
template <typename A, typename B> struct pick_t<false, A, B> { using type = B; };

template <typename A, typename B> struct same_t { static constexpr bool value = false; };
template <typename A> struct same_t<A, A> { static constexpr bool value = true; };

__device__ __forceinline__ float as_f32(uint32_t bits) { return __builtin_bit_cast(float, bits); }
__device__ __forceinline__ uint32_t as_u32(float v) { return __builtin_bit_cast(uint32_t, v); }

template <typename T> __device__ __forceinline__ float widen(T v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T narrow(float v) { return static_cast<T>(v); }
// float -> T -> float: the value a tensor of type T would hold.
template <typename T> __device__ __forceinline__ float round_through(float v) {
    if constexpr (same_t<T, float>::value) return v;
    else return static_cast<float>(static_cast<T>(v));
}

// round_through<T> on every element of an array.  gfx950 rounds two floats to a bf16 pair in one instruction
// (v_cvt_pk_bf16_f32); element by element the compiler spends one such instruction per value, pair by pair half as
// many - same rounding, same results.
template <typename T, int N> __device__ __forceinline__ void round_through_all(float (&v)[N]) {
    if constexpr (same_t<T, float>::value) {
        return;
    } else if constexpr (same_t<T, bf16>::value && N % 2 == 0) {
        using float2v = vec_t<float, 2>;
        using bf16x2 = vec_t<bf16, 2>;
#pragma unroll
        for (int i = 0; i < N; i += 2) {
            const float2v pair = {v[i], v[i + 1]};
            const float2v back = __builtin_convertvector(__builtin_convertvector(pair, bf16x2), float2v);
            v[i] = back.x;
            v[i + 1] = back.y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = round_through<T>(v[i]);
    }
}

// narrow<T> of every element, pair by pair for bf16 for the same reason: the pair comes out packed in one register.
template <typename T, int N> __device__ __forceinline__ void narrow_all(const float (&v)[N], T (&out)[N]) {
    if constexpr (same_t<T, bf16>::value && N % 2 == 0) {
        using float2v = vec_t<float, 2>;
        using bf16x2 = vec_t<bf16, 2>;
#pragma unroll
        for (int i = 0; i < N; i += 2) {
            const float2v pair = {v[i], v[i + 1]};
            const bf16x2 packed = __builtin_convertvector(pair, bf16x2);
            out[i] = packed.x;
            out[i + 1] = packed.y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) out[i] = narrow<T>(v[i]);
    }
}

// ---- N-element contiguous load / store --------------------------------------
template <typename T, int N, int MODE>
__device__ __forceinline__ void load_vec(const T *__restrict__ p, T (&dst)[N]) {
    if constexpr (MODE != kScalar) {
        using V = vec_t<T, N>;
        V v;
        if constexpr (MODE == kStream) v = __builtin_nontemporal_load(reinterpret_cast<const V *>(p));
        else v = *reinterpret_cast<const V *>(p);
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = v[i];
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = p[i];
    }
}

template <typename T, int N, int MODE>
__device__ __forceinline__ void store_vec(T *__restrict__ p, const T (&src)[N]) {
    if constexpr (MODE != kScalar) {
        using V = vec_t<T, N>;
        V v;
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = src[i];
        if constexpr (MODE == kStream) __builtin_nontemporal_store(v, reinterpret_cast<V *>(p));
        else *reinterpret_cast<V *>(p) = v;
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) p[i] = src[i];
    }
}

// Loads / stores N elements as ceil(N*sizeof(T)/16) instructions of at most 16 bytes.
template <typename T, int N, int MODE>
__device__ __forceinline__ void load_wide(const T *__restrict__ p, T (&dst)[N]) {
    constexpr int PER = 16 / sizeof(T);
    if constexpr (N <= PER) {
        load_vec<T, N, MODE>(p, dst);
    } else {
        static_assert(N % PER == 0, "whole 16-byte pieces");
#pragma unroll
        for (int k = 0; k < N / PER; ++k) {
            T piece[PER];
            load_vec<T, PER, MODE>(p + k * PER, piece);
#pragma unroll
            for (int i = 0; i < PER; ++i) dst[k * PER + i] = piece[i];
        }
    }
}

template <typename T, int N, int MODE>
__device__ __forceinline__ void store_wide(T *__restrict__ p, const T (&src)[N]) {
    constexpr int PER = 16 / sizeof(T);
    if constexpr (N <= PER) {
        store_vec<T, N, MODE>(p, src);
    } else {
        static_assert(N % PER == 0, "whole 16-byte pieces");
#pragma unroll
        for (int k = 0; k < N / PER; ++k) {
            T piece[PER];
#pragma unroll
            for (int i = 0; i < PER; ++i) piece[i] = src[k * PER + i];
            store_vec<T, PER, MODE>(p + k * PER, piece);
        }
    }
}

// ---- buffer addressing ---------------------------------------------------------
// A descriptor over [base, base + bytes) held in scalar registers.  Loads and stores through it take a 32-bit
// byte offset per lane, so a wavefront spends no vector instructions on 64-bit addresses before its first load
// is out (on shard-sized launches, which are all ramp, that measured 6-9 % of the kernel), and an access past
// `bytes` is dropped by the hardware instead of faulting.  The interior blocks of the kernels build one
// descriptor per stream over the block's own span.
using buffer_t = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ buffer_t buffer_over(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, static_cast<int>(bytes), 0x00020000);
}
// Cache policy operand of the buffer instructions: plain, the non-temporal bit, or (stores) the sc1 bit, which
// makes a store write through the XCD's L2 instead of leaving a dirty line for a later eviction.
constexpr int kCached = 0, kNtBit = 2, kSc1Bit = 16;
template <int MODE> constexpr int policy_of() { return MODE >= kStream ? kNtBit : kCached; }

using u32x2 = vec_t<uint32_t, 2>;
using u32x4 = vec_t<uint32_t, 4>;

// N elements of T (4, 8 or 16 bytes, or a multiple of 16) at byte offset `at`.
template <typename T, int N, int POLICY>
__device__ __forceinline__ void buffer_load(buffer_t b, uint32_t at, T (&dst)[N]) {
    constexpr int BYTES = N * sizeof(T);
    static_assert(BYTES == 4 || BYTES == 8 || BYTES % 16 == 0, "whole dwords");
    using V = vec_t<T, N>;
    if constexpr (BYTES == 4) {
        const uint32_t w = __builtin_amdgcn_raw_buffer_load_b32(b, at, 0, POLICY);
        const V v = __builtin_bit_cast(V, w);
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = v[i];
    } else if constexpr (BYTES == 8) {
        const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(b, at, 0, POLICY);
        const V v = __builtin_bit_cast(V, w);
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = v[i];
    } else {
        constexpr int PER = 16 / sizeof(T);
        using P = vec_t<T, PER>;
#pragma unroll
        for (int k = 0; k < BYTES / 16; ++k) {
            const u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(b, at + 16 * k, 0, POLICY);
            const P v = __builtin_bit_cast(P, w);
#pragma unroll
            for (int i = 0; i < PER; ++i) dst[k * PER + i] = v[i];
        }
    }
}

template <typename T, int N, int POLICY>
__device__ __forceinline__ void buffer_store(buffer_t b, uint32_t at, const T (&src)[N]) {
    constexpr int BYTES = N * sizeof(T);
    static_assert(BYTES == 4 || BYTES == 8 || BYTES % 16 == 0, "whole dwords");
    using V = vec_t<T, N>;
    if constexpr (BYTES == 4) {
        V v;
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = src[i];
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), b, at, 0, POLICY);
    } else if constexpr (BYTES == 8) {
        V v;
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = src[i];
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), b, at, 0, POLICY);
    } else {
        constexpr int PER = 16 / sizeof(T);
        using P = vec_t<T, PER>;
#pragma unroll
        for (int k = 0; k < BYTES / 16; ++k) {
            P v;
#pragma unroll
            for (int i = 0; i < PER; ++i) v[i] = src[k * PER + i];
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), b, at + 16 * k, 0, POLICY);
        }
    }
}

// ---- max over LANES adjacent lanes (LANES in {1,2,4,8,16}) -------------------
// DPP butterflies inside one 16-lane row: quad permutes for xor 1 / xor 2, then
// row_half_mirror and row_mirror, which act as xor 4 / xor 8 once the quads
// (resp. halves) already agree.  Every lane of the group ends with the maximum.
// Operates on the bit patterns of non-negative floats, where unsigned integer
// order equals float order and a NaN pattern exceeds +Inf, so a NaN anywhere in
// the group wins the reduction - the behaviour of torch.amax.
template <int CTRL> __device__ __forceinline__ uint32_t dpp_max_step(uint32_t v) {
    // old value 0 with bound_ctrl set: 0 is the identity of an unsigned maximum, which lets the compiler fold the
    // lane permutation into the maximum itself (one v_max_u32 with a DPP operand per step instead of a copy, a
    // permuting move, two wait states and the maximum).  Every lane has a valid source under these permutations.
    uint32_t other = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xF, 0xF, true));
    return other > v ? other : v;
}

template <int LANES> __device__ __forceinline__ uint32_t group_max_bits(uint32_t v) {
    static_assert(LANES == 1 || LANES == 2 || LANES == 4 || LANES == 8 || LANES == 16, "row-sized groups only");
    if constexpr (LANES >= 2) v = dpp_max_step<0xB1>(v);   // quad_perm [1,0,3,2]
    if constexpr (LANES >= 4) v = dpp_max_step<0x4E>(v);   // quad_perm [2,3,0,1]
    if constexpr (LANES >= 8) v = dpp_max_step<0x141>(v);  // row_half_mirror
    if constexpr (LANES >= 16) v = dpp_max_step<0x140>(v); // row_mirror
    return v;
}

// scale = max(absmax / 127, 2^-23), bit-identical to an IEEE division.
// absmax/127 is evaluated as q0 = a*c, r = fma(-q0, 127, a), q1 = fma(r, c, q0)
// with c = RN(1/127): an exhaustive sweep over every finite non-negative float
// shows q1 == RN(a/127) (tests/native/check_scale127.c).  +Inf would turn the
// residual into NaN and is passed through; a NaN absmax stays NaN because the
// final comparison is false, matching torch.clamp(min=eps).
__device__ __forceinline__ float scale_from_absmax(float absmax) {
    const float c = as_f32(0x3C010204u);
    const float q0 = absmax * c;
    const float r = __builtin_fmaf(-q0, 127.0f, absmax);
    float s = __builtin_fmaf(r, c, q0);
    s = as_u32(absmax) == 0x7F800000u ? absmax : s;
    return s < as_f32(kEpsBits) ? as_f32(kEpsBits) : s;
}

// Bit pattern of the largest magnitude in the group that the VEC values of LPG adjacent lanes form; every lane gets it.
template <int VEC, int LPG>
__device__ __forceinline__ uint32_t group_absmax_bits(const float (&p)[VEC]) {
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        const uint32_t a = as_u32(p[i]) & 0x7FFFFFFFu;
        m = a > m ? a : m;
    }
    return group_max_bits<LPG>(m);
}

// (For a pure 16-bit tensor the lane's maximum could be taken on pairs of 16-bit magnitudes before widening,
// v_pk_max_u16, half the instructions of this loop.  Measured: 2 % slower at every size, 26 M bf16 elements 14.7
// against 14.4 us - the kernel waits on memory, and the packed chain is longer.  Not used.)

// Scale of that group.
template <int VEC, int LPG>
__device__ __forceinline__ float group_scale(const float (&p)[VEC]) {
    return scale_from_absmax(as_f32(group_absmax_bits<VEC, LPG>(p)));
}

// Value of lane K of the caller's quad (four adjacent lanes), in every lane of the quad.
template <int K> __device__ __forceinline__ float quad_broadcast(float v) {
    return as_f32(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(as_u32(v)), K * 0x55, 0xF, 0xF, true)));
}

__device__ __forceinline__ int cvt_i32(float v) {  // NaN -> 0, saturating
    int c;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(c) : "v"(v));
    return c;
}

// v[i] = T(v[i] / divisor) for a divisor that is the same for the whole grid (the mean of a reduction).  When the
// divisor is a power of two whose reciprocal is a normal float - the usual world sizes - the product with that
// reciprocal is taken instead: both are the correctly rounded value of the same real number, so the bits agree for
// every input, and the division's ten-odd instructions per element become one.
template <typename T, int N> __device__ __forceinline__ void divide_all(float (&v)[N], float divisor) {
    const uint32_t bits = as_u32(divisor);
    const uint32_t exponent = bits >> 23;                  // the sign bit is part of it: positive divisors only
    if ((bits & 0x007FFFFFu) == 0 && exponent >= 2 && exponent <= 252) {
        const float reciprocal = as_f32((254u - exponent) << 23);
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = v[i] * reciprocal;
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = v[i] / divisor;
    }
    round_through_all<T, N>(v);
}

// codes[i] = rint(p[i] / scale) as the reference computes it (IEEE division, then round-half-even), a NaN
// quotient -> 0.  A code comes back as the bit pattern of (code + 1.5 * 2^23): its low byte is the int8 code that
// goes into the payload (pack4 takes low bytes), and code_value() gives the integer back as a float.
//
// The path has no division per element and no data-dependent branch.  y = 1/scale is one IEEE division per lane,
// i.e. the correctly rounded reciprocal; per element q0 = p*y is within an ulp and a half of p/scale,
// r = fma(-q0, scale, p) is its exact remainder, and q1 = fma(r, y, q0) is Markstein's correction step for division
// with a fused multiply-add: RN(q + d) for the real quotient q and a |d| below 2^-23 ulp.  Markstein's theorem
// promises q1 = RN(q) only for a q0 within one ulp, so the claim that matters here - rint(q1) is the code the
// division gives - is checked, not inferred: q1 and RN(q) are equal or neighbouring floats and every half-integer
// up to 127.5 is a float, so the codes can differ only for a p within a few ulps of (k + 0.5) * scale, and the
// operations are invariant under a common power of two away from underflow.  tests/native/quotient_check.hip walks
// all 2^23 scale mantissas x 256 half-integers x 13 neighbouring dividends at three exponents (8*10^10 pairs, every
// such case) and 2.6*10^10 sampled pairs over the whole exponent range 2^-23 .. 2^120, among them dividends with 8
// or 11 significant bits: no code and no quotient differs.  The one case outside, a remainder that underflows,
// needs |p/scale| < 2^-64, where the code is 0 whatever the last bit of the quotient is.  The ragged edge uses
// the same operations (encode below), so an element's code does not depend on the block it falls into.
// (A reciprocal-multiply fast path with a fallback
// for quotients next to a tie, which this replaces, took the fallback in most wavefronts of a 16-bit tensor -
// 127*x/absmax hits exact ties all the time when x and absmax have 8-bit mantissas - and ran it 25 % slower.)
// Adding 1.5 * 2^23 rounds q1 to an integer, half to even, and leaves it in the low mantissa bits.
//
// No +-127 clamp is needed: |p| <= absmax and scale >= RN(absmax/127), hence |p/scale| <= 127 * (1 + 2^-23) and
// the rounded quotient is at most 127.  A scale that is not finite (a NaN or an Inf in the group) makes every
// quotient of the group 0 or NaN: all of its codes are 0.
constexpr float kCodeMagic = 12582912.0f;   // 1.5 * 2^23

__device__ __forceinline__ float code_value(int code_bits) { return as_f32(static_cast<uint32_t>(code_bits)) - kCodeMagic; }

// Inf or NaN scale: every code of the group is 0.
__device__ __forceinline__ bool scale_not_finite(float scale) { return (as_u32(scale) & 0x7F800000u) == 0x7F800000u; }

// The codes of a group whose scale is finite; for any other scale the caller must discard them (encode_group
// does it per element; a caller that only packs them can zero whole words instead, one select per four codes).
// `y` is the correctly rounded reciprocal of `scale` (an IEEE division 1/scale).
template <int N>
__device__ __forceinline__ void encode_group_finite(const float (&p)[N], float scale, float y, int (&codes)[N]) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const float q0 = p[i] * y;
        const float r = __builtin_fmaf(-q0, scale, p[i]);
        codes[i] = static_cast<int>(as_u32(__builtin_fmaf(r, y, q0) + kCodeMagic));
    }
}

template <int N>
__device__ __forceinline__ void encode_group(const float (&p)[N], float scale, float y, int (&codes)[N]) {
    const bool no_codes = scale_not_finite(scale);   // one compare per lane
    encode_group_finite<N>(p, scale, y, codes);
#pragma unroll
    for (int i = 0; i < N; ++i) codes[i] = no_codes ? static_cast<int>(as_u32(kCodeMagic)) : codes[i];
}

template <int N>
__device__ __forceinline__ void encode_group(const float (&p)[N], float scale, int (&codes)[N]) {
    encode_group<N>(p, scale, 1.0f / scale, codes);
}

// Single-element form for the ragged edge: the same operations as encode_group, so that an element gets the same
// code whether it falls into an interior block or into the tail.
__device__ __forceinline__ int encode(float p, float scale) {
    const float one[1] = {p};
    int bits[1];
    encode_group<1>(one, scale, bits);
    return static_cast<int>(code_value(bits[0]));   // an integer in [-127, 127]: the conversion is exact
}

// Low bytes of four ints -> one little-endian word (three v_perm_b32).
__device__ __forceinline__ uint32_t pack4(int c0, int c1, int c2, int c3) {
    const uint32_t lo = __builtin_amdgcn_perm(static_cast<uint32_t>(c1), static_cast<uint32_t>(c0), 0x0C0C0400u);
    const uint32_t hi = __builtin_amdgcn_perm(static_cast<uint32_t>(c3), static_cast<uint32_t>(c2), 0x04000C0Cu);
    return lo | hi;
}

// signed byte k of a packed word -> float
__device__ __forceinline__ float code_to_float(uint32_t word, int k) {
    return static_cast<float>(static_cast<int>(static_cast<int8_t>(word >> (8 * k))));
}

}  // namespace lbc
