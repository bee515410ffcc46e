// Device-side helpers shared by the gfx950 codec kernels: 16-bit float types,
// vector load/store, wavefront-row (DPP) reductions and the exact arithmetic
// primitives the wire format depends on.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lbc {

using f16 = _Float16;
using bf16 = __bf16;

constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr uint32_t kEpsBits = 0x34000000u;  // 2^-23, torch.finfo(float32).eps

template <typename T, int N>
using vec_t = T __attribute__((ext_vector_type(N)));

template <typename T> struct is_void_t { static constexpr bool value = false; };
template <> struct is_void_t<void> { static constexpr bool value = true; };

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

// ---- N-element contiguous load / store --------------------------------------
// ALIGNED: one vector instruction (the caller guarantees N*sizeof(T) alignment);
// otherwise element by element.
template <typename T, int N, bool ALIGNED>
__device__ __forceinline__ void load_vec(const T *__restrict__ p, T (&dst)[N]) {
    if constexpr (ALIGNED) {
        using V = vec_t<T, N>;
        V v = *reinterpret_cast<const V *>(p);
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = v[i];
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = p[i];
    }
}

template <typename T, int N, bool ALIGNED>
__device__ __forceinline__ void store_vec(T *__restrict__ p, const T (&src)[N]) {
    if constexpr (ALIGNED) {
        using V = vec_t<T, N>;
        V v;
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = src[i];
        *reinterpret_cast<V *>(p) = v;
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) p[i] = src[i];
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
    uint32_t other = static_cast<uint32_t>(
        __builtin_amdgcn_update_dpp(static_cast<int>(v), static_cast<int>(v), CTRL, 0xF, 0xF, false));
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

// scale = max(absmax / 127, 2^-23) with a true IEEE division; a NaN absmax
// stays NaN (the comparison is false), matching torch.clamp(min=eps).
__device__ __forceinline__ float scale_from_absmax(float absmax) {
    float s = absmax / 127.0f;
    return s < as_f32(kEpsBits) ? as_f32(kEpsBits) : s;
}

// code = saturate(rint(p / scale)) with NaN -> 0.  rintf is round-half-even
// (v_rndne_f32); the float -> int conversion instruction returns 0 for NaN and
// saturates infinities, after which the integer clamp applies +-127.
__device__ __forceinline__ int encode(float p, float scale) {
    float q = __builtin_rintf(p / scale);
    int c;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(c) : "v"(q));
    c = c < -127 ? -127 : c;
    return c > 127 ? 127 : c;
}

__device__ __forceinline__ uint32_t pack4(int c0, int c1, int c2, int c3) {
    return (static_cast<uint32_t>(c0) & 0xFFu) | ((static_cast<uint32_t>(c1) & 0xFFu) << 8) |
           ((static_cast<uint32_t>(c2) & 0xFFu) << 16) | (static_cast<uint32_t>(c3) << 24);
}

// signed byte k of a packed word -> float
__device__ __forceinline__ float code_to_float(uint32_t word, int k) {
    return static_cast<float>(static_cast<int>(static_cast<int8_t>(word >> (8 * k))));
}

}  // namespace lbc
