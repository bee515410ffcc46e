// Byte layout and small arithmetic helpers shared by the kernels that read and write the payload
// format of the reference's CUDA extension (cuda_wire.hip, cuda_wire_general.hip).
#pragma once
#include "device_utils.h"

namespace lbc {

constexpr int kPlain = 0, kNonTemporal = 1;

// N 32-bit words at an address aligned to ALIGN bytes.
template <int N, int ALIGN> struct words_at {
    typedef vec_t<uint32_t, N> type __attribute__((aligned(ALIGN)));
};

template <int N, int ALIGN, int NT>
__device__ __forceinline__ void load_words(const uint8_t *p, uint32_t (&w)[N]) {
    using V = typename words_at<N, ALIGN>::type;
    vec_t<uint32_t, N> v;
    if constexpr (NT == kNonTemporal) v = __builtin_nontemporal_load(reinterpret_cast<const V *>(p));
    else v = *reinterpret_cast<const V *>(p);
#pragma unroll
    for (int i = 0; i < N; ++i) w[i] = v[i];
}

template <int N, int ALIGN, int NT>
__device__ __forceinline__ void store_words(uint8_t *p, const uint32_t (&w)[N]) {
    using V = typename words_at<N, ALIGN>::type;
    vec_t<uint32_t, N> v;
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = w[i];
    if constexpr (NT == kNonTemporal) __builtin_nontemporal_store(v, reinterpret_cast<V *>(p));
    else *reinterpret_cast<V *>(p) = v;
}

// VEC elements of T at an address aligned to sizeof(T) only.
template <typename T, int VEC, int NT>
__device__ __forceinline__ void load_elems(const T *p, T (&dst)[VEC]) {
    typedef vec_t<T, VEC> V __attribute__((aligned(sizeof(T))));
    vec_t<T, VEC> v;
    if constexpr (NT == kNonTemporal) v = __builtin_nontemporal_load(reinterpret_cast<const V *>(p));
    else v = *reinterpret_cast<const V *>(p);
#pragma unroll
    for (int i = 0; i < VEC; ++i) dst[i] = v[i];
}

template <typename T, int VEC, int NT>
__device__ __forceinline__ void store_elems(T *p, const T (&src)[VEC]) {
    typedef vec_t<T, VEC> V __attribute__((aligned(sizeof(T))));
    vec_t<T, VEC> v;
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = src[i];
    if constexpr (NT == kNonTemporal) __builtin_nontemporal_store(v, reinterpret_cast<V *>(p));
    else *reinterpret_cast<V *>(p) = v;
}

// Compact 16-bit payloads have a group pitch of 66 bytes (64 codes, a 2-byte scale), so a lane's 8 code bytes
// start at an address that is only 2-byte aligned, and a misaligned 8-byte access runs at a fraction of the
// aligned rate.  This reads the aligned 12-byte window that contains them instead and shifts the piece out:
// at == 0 mod 4: window [at, at + 12); at == 2 mod 4: window [at - 2, at + 10).  `after` receives the two bytes
// that follow the piece - for the lane that owns the last piece of a group, the group's scale - so the scales
// need no loads of their own.  `b` covers the payload from a 4-byte aligned address on, up to window_span() of
// its last byte, and `at` is relative to it.  The span is rounded up to whole dwords because the hardware drops a
// dword that is only partly inside a buffer, and the last dword of an odd number of groups holds the last scale;
// the two bytes read past the payload share an aligned dword, hence a page, with that scale.  Whole dwords past
// the span read as zero (only ever the unused tail of a window).
__device__ __forceinline__ uint32_t window_span(uint32_t bytes) { return (bytes + 3u) & ~3u; }

template <int POLICY>
__device__ __forceinline__ void load_piece16(buffer_t b, uint32_t at, uint32_t (&words)[2], uint32_t &after) {
    const uint32_t odd = at & 2u;
    const vec_t<uint32_t, 3> w = __builtin_amdgcn_raw_buffer_load_b96(b, at - odd, 0, POLICY);
    const uint32_t shift = odd * 8u;
    words[0] = __builtin_amdgcn_alignbit(w[1], w[0], shift);
    words[1] = __builtin_amdgcn_alignbit(w[2], w[1], shift);
    after = odd ? w[2] >> 16 : w[2] & 0xFFFFu;
}

// Cache policy of those windows.  Measured on the W=8 reduce of 26.2 M bf16 elements: windows 45.9 us with the
// non-temporal hint, 47.6 us without, against 50.0 us for misaligned 8-byte loads plus a 2-byte load per scale
// (and 55.9 us when the runs are staged through LDS with aligned 16-byte loads: the barrier costs more than the
// misalignment).  Few payloads: the output dominates and cached payload loads are the faster ones, as in the
// other layouts.
template <int NT, int WORLD> constexpr int window_policy() { return NT == kNonTemporal && WORLD >= 4 ? kNtBit : kCached; }

// Stores to such positions are misaligned 8-byte stores in most kernels.  Splitting one into short, aligned dword,
// short made the ring's gather hop 30 % slower (56.5 against 43.0 us on 52 M bf16 elements).  What pays, on the
// gather hop of large chunks and together with the non-temporal hint, is to shift the bytes across lanes instead: a DPP row holds two groups, lanes 0-7 the even one, whose codes start on a dword when the payload
// does, and lanes 8-15 the odd one, whose 66 bytes start two bytes into a dword.  The pair is 33 dwords:
//   D[0..15]  the even group's codes, two dwords a lane, as they are;
//   D[16+j], j = 0..15: the odd group's code dwords moved up by two bytes, alignbit(in[j], in[j - 1], 16), where
//             in[-1] is the even group's scale in its upper half - so D[16] carries that scale;
//   D[32]     the odd group's last two code bytes and its scale.
// in[j - 1] is the lane's own first dword or the second dword of the lane before it (row_shr:1).  Every lane of the
// row must call this (live or not); `pair` points at the even group's codes and is 4-byte aligned; `scale` is the
// group's 16-bit scale, the same in its eight lanes; when the odd group lies past the end, the even group's scale is
// written by itself.
template <int POLICY>
__device__ __forceinline__ void store_group_pair16(uint8_t *pair, int lane, const uint32_t (&words)[2], uint32_t scale, bool live,
                                                   bool odd_group_live) {
    const int row_lane = lane & 15, l = row_lane & 7;
    const bool odd = (row_lane & 8) != 0;
    const uint32_t before = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(words[1]), 0x111, 0xF, 0xF, true));
    const uint32_t even_scale = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(scale), 0x118, 0xF, 0xF, true));
    const uint32_t previous = l == 0 ? even_scale << 16 : before;
    uint32_t out[2] = {words[0], words[1]};
    if (odd) {
        out[0] = __builtin_amdgcn_alignbit(words[0], previous, 16);
        out[1] = __builtin_amdgcn_alignbit(words[1], words[0], 16);
    }
    if (!live) return;
    store_words<2, 4, POLICY>(pair + (odd ? 64 : 0) + 8 * l, out);
    if (row_lane == 15) *reinterpret_cast<uint32_t *>(pair + 128) = (words[1] >> 16) | (scale << 16);
    if (row_lane == 0 && !odd_group_live) *reinterpret_cast<uint16_t *>(pair + 64) = static_cast<uint16_t>(scale);
}

// The value lane 7 (lanes 0-7) or lane 15 (lanes 8-15) of the caller's row holds: the last lane of an 8-lane group.
__device__ __forceinline__ uint32_t from_last_lane_of_8(uint32_t v, bool upper_half) {
    const uint32_t low = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x150 + 7, 0xF, 0xF, true));
    const uint32_t high = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x150 + 15, 0xF, 0xF, true));
    return upper_half ? high : low;
}

template <typename T, int BIT = 8> struct wire {
    static constexpr int ITEM = sizeof(T);
    static constexpr int VEC = 16 / ITEM;                  // elements per lane: 16 bytes of the tensor
    static constexpr int CODE_BYTES = VEC * BIT / 8;        // 8, 4 or (4-bit codes of an fp32 tensor) 2
    static constexpr int WORDS = CODE_BYTES >= 4 ? CODE_BYTES / 4 : 1;   // 32-bit registers holding them
    static constexpr int TILE = kWave * VEC;
    static constexpr float LEVELS = BIT == 8 ? 127.0f : 7.0f;
};

// Byte position of element k (0..3) inside its 32-bit word: fp32 payloads reverse all four
// bytes, 16-bit payloads swap byte pairs.
template <typename T> __device__ __forceinline__ constexpr int byte_in_word(int k) {
    return sizeof(T) == 4 ? 3 - k : (k ^ 1);
}
// Byte position of element k of a group inside the group's code bytes.
template <typename T> __device__ __forceinline__ int byte_in_group(int k) {
    constexpr int ITEM = sizeof(T);
    return (k / ITEM) * ITEM + (ITEM - 1 - k % ITEM);
}

// COMPACT payloads interleave [G code bytes][scale] per group, so a 128-byte line is shared by
// neighbouring wavefront instructions and payload accesses must stay cacheable even when the tensors
// stream with the non-temporal hint (the hint would drop the line between its two uses).  Otherwise
// the policy measured for the portable format applies: code stores follow the tensors' hint, code
// loads are non-temporal only from four payloads on.
template <typename T, int G, bool COMPACT, int BIT = 8> struct group_layout {
    static constexpr int ITEM = sizeof(T);
    static constexpr int CB = G * BIT / 8;      // code bytes per group
    const int64_t groups;
    __device__ __forceinline__ int64_t codes(int64_t group) const { return COMPACT ? group * (CB + ITEM) : group * CB; }
    __device__ __forceinline__ int64_t scale(int64_t group) const {
        return COMPACT ? group * (CB + ITEM) + CB : groups * CB + group * ITEM;
    }
};

// The VEC codes of one lane -> its 32-bit words, in the byte / nibble order of the format.
template <typename T, int BIT, int VEC, int WORDS>
__device__ __forceinline__ void pack_codes(const int (&c)[VEC], uint32_t (&words)[WORDS]) {
    if constexpr (BIT == 8) {
#pragma unroll
        for (int k = 0; k < WORDS; ++k) {
            if constexpr (sizeof(T) == 4) words[k] = pack4(c[4 * k + 3], c[4 * k + 2], c[4 * k + 1], c[4 * k]);
            else words[k] = pack4(c[4 * k + 1], c[4 * k], c[4 * k + 3], c[4 * k + 2]);
        }
    } else {
        // Four codes make one 16-bit unit with the first code on top.  A 16-bit tensor's lane holds two
        // such units, low half first; an fp32 tensor's lane holds one (half of a 32-bit payload word).
        static_assert(WORDS == 1 && (VEC == 8 || VEC == 4), "a 4-bit lane owns at most one register");
        uint32_t word = 0;
#pragma unroll
        for (int i = 0; i < VEC; ++i)
            word |= (static_cast<uint32_t>(c[i]) & 0xFu) << (16 * (i / 4) + 12 - 4 * (i % 4));
        words[0] = word;
    }
}

// Byte offset, inside a group's code bytes, of the piece owned by the lane whose first element is k0.
// An fp32 payload word holds eight 4-bit codes, elements 0-3 in its upper half: the two lanes sharing a
// word write its halves swapped, which keeps a wavefront's 2-byte accesses one contiguous run.
template <typename T, int BIT> __device__ __forceinline__ int piece_offset(int k0) {
    if constexpr (BIT == 4 && sizeof(T) == 4) return (k0 / 8) * 4 + ((k0 & 4) ? 0 : 2);
    else return k0 * BIT / 8;
}

template <typename T, int BIT, int PNT, int WORDS>
__device__ __forceinline__ void store_piece(uint8_t *p, const uint32_t (&words)[WORDS]) {
    if constexpr (wire<T, BIT>::CODE_BYTES == 2) *reinterpret_cast<uint16_t *>(p) = static_cast<uint16_t>(words[0]);
    else store_words<WORDS, sizeof(T), PNT>(p, words);
}

template <typename T, int BIT, int PNT, int WORDS>
__device__ __forceinline__ void load_piece(const uint8_t *p, uint32_t (&words)[WORDS]) {
    if constexpr (wire<T, BIT>::CODE_BYTES == 2) words[0] = *reinterpret_cast<const uint16_t *>(p);
    else load_words<WORDS, sizeof(T), PNT>(p, words);
}

// Code i of the lane's words as a float.
template <typename T, int BIT, int WORDS>
__device__ __forceinline__ float unpack_code(const uint32_t (&words)[WORDS], int i) {
    if constexpr (BIT == 8) {
        return code_to_float(words[i / 4], byte_in_word<T>(i % 4));
    } else {
        const int top = 16 - 16 * (i / 4) + 4 * (i % 4);   // left shift that puts the nibble on top
        return static_cast<float>(static_cast<int32_t>(words[0] << top) >> 28);
    }
}

// Code of element k of a group read from the group's code bytes (ragged-edge path).
template <typename T, int BIT> __device__ __forceinline__ float code_at(const uint8_t *group_codes, int k) {
    if constexpr (BIT == 8) {
        return static_cast<float>(static_cast<int8_t>(group_codes[byte_in_group<T>(k)]));
    } else {
        constexpr int ITEM = sizeof(T), PER_WORD = 2 * ITEM;
        const int in_word = k % PER_WORD;
        const uint32_t byte = group_codes[(k / PER_WORD) * ITEM + (ITEM - 1 - in_word / 2)];
        const uint32_t nibble = (in_word & 1) ? (byte & 0xFu) : (byte >> 4);
        return static_cast<float>(static_cast<int32_t>(nibble << 28) >> 28);
    }
}

// float(scale) / levels with IEEE rounding.
template <int BIT> __device__ __forceinline__ float step_of(float stored);

template <bool COMPACT, int NT, int WORLD> constexpr int payload_load_hint() { return COMPACT || WORLD < 4 ? kPlain : NT; }

// float(scale) / 127 with IEEE rounding: the three-operation form proven exhaustively for
// every finite float (tests/native/check_scale127.c); an infinite scale passes through.
static __device__ __forceinline__ float div127(float a) {
    const float c = as_f32(0x3C010204u);
    const float q0 = a * c;
    const float r = __builtin_fmaf(-q0, 127.0f, a);
    const float q = __builtin_fmaf(r, c, q0);
    return (as_u32(a) & 0x7FFFFFFFu) == 0x7F800000u ? a : q;
}

template <> __device__ __forceinline__ float step_of<8>(float stored) { return div127(stored); }
template <> __device__ __forceinline__ float step_of<4>(float stored) { return stored / 7.0f; }

// a + b as a native add in T returns it, for a and b that are values of T.  The fp32 sum converted to T is that
// result: fp32's 24 significand bits are at least 2p + 2 for fp16 (p = 11) and bfloat16 (p = 8), so the conversion
// never meets a value the fp32 add has moved onto or off a rounding boundary of T.  Checked for every pair of finite
// values of both types by tests/native/check_half_sum.c.
template <typename T> __device__ __forceinline__ float add_in(float a, float b) { return round_through<T>(a + b); }

// ---- elements as stored (bit patterns), for the kernels that must keep NaN payloads and compare magnitudes ----
template <typename T> struct raw_bits;
template <> struct raw_bits<float> { using type = uint32_t; static constexpr uint32_t ABS = 0x7FFFFFFFu, INF = 0x7F800000u; };
template <> struct raw_bits<f16> { using type = uint16_t; static constexpr uint32_t ABS = 0x7FFFu, INF = 0x7C00u; };
template <> struct raw_bits<bf16> { using type = uint16_t; static constexpr uint32_t ABS = 0x7FFFu, INF = 0x7F80u; };

template <typename T> __device__ __forceinline__ float value_of(uint32_t raw) {
    return widen(__builtin_bit_cast(T, static_cast<typename raw_bits<T>::type>(raw)));
}
template <typename T> __device__ __forceinline__ uint32_t raw_from(float v) {
    return __builtin_bit_cast(typename raw_bits<T>::type, narrow<T>(v));
}

// First element of a group's scan in the reference's one-thread-per-group kernels: 0 for fp32 tensors,
// rotated by shared-memory bank for 16-bit ones (quant_kernel.cuh:30-32).
template <typename T, int G> __device__ __forceinline__ int scan_start(int64_t group) {
    if constexpr (sizeof(T) == 4) return 0;
    else return 4 * static_cast<int>((group & 31) / (32 / (G / 4)));
}


// The reference's general kernels take a group's maximum as a running `(m > a) ? m : a` over the group's
// scan (utils.cuh:11-14, quant_kernel_fp32.cuh:93-97, quant_kernel.cuh:33-38): a NaN replaces the maximum and
// the next element replaces the NaN, so the result is the maximum of what follows the group's last NaN, or that
// NaN when it ends the scan.  `mag` are the magnitude bits of the lane's elements as stored, `k0` the lane's
// first element inside its group, `start` the element the scan begins at.  Returns the scale as stored.
// `any_nan` (optional) receives whether any lane of the wavefront holds a NaN.
template <typename T, int G, int VEC>
__device__ __forceinline__ uint32_t running_max_raw(const uint32_t (&mag)[VEC], int k0, int start, bool *any_nan = nullptr) {
    constexpr int LPG = G / VEC;
    using RB = raw_bits<T>;
    // A NaN's magnitude bits lie above those of every number, so the lane's plain maximum says whether it holds one.
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) m = mag[i] > m ? mag[i] : m;
    const bool nans = __ballot(m > RB::INF) != 0;   // wavefront-uniform, rare
    if (any_nan) *any_nan = nans;
    if (nans) {
        uint32_t last = 0;          // 1 + scan position of the group's last NaN
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const uint32_t pos = static_cast<uint32_t>(k0 + i - start) & (G - 1);
            if (mag[i] > RB::INF && pos + 1 > last) last = pos + 1;
        }
        last = group_max_bits<LPG>(last);
        const uint32_t from = last == G ? G - 1 : last;
        m = 0;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const uint32_t pos = static_cast<uint32_t>(k0 + i - start) & (G - 1);
            if (pos >= from && mag[i] > m) m = mag[i];
        }
    }
    return group_max_bits<LPG>(m);
}

}  // namespace lbc
