// Kernels for the payload format of the reference's CUDA extension (ccdl_cuda_ops), so that
// gfx950 ranks can exchange payloads with ranks running that extension.
//
// Format (ccdl_comm/csrc/quantization/quant_pack_kernel.cu:101-162 writes it,
// dequant_reduce_kernel.cu:27-69 reads it), for element type T of the tensor:
//   scale of a group  = max |p| over the group, stored as T (NaNs skipped, fmaxf);
//   code              = rint(p * (127 / max(float(scale), 1e-6f))), NaN -> 0;
//   bytes of a group  = codes with the byte order reversed inside every sizeof(T)-byte word
//                       (2-byte words for fp16/bf16, 4-byte words for fp32);
//   compact layout    = per group [G code bytes][scale]; otherwise all code bytes, then all scales;
//   decode            = float(code) * (float(scale) / 127), rounded to T.
// 4-bit codes (BIT = 4; quant_pack_kernel.cu:103,120-130,145-158, inner.cuh:36-40): multiplier
// 7 / max(scale, 1e-6), two's-complement nibbles, 2*sizeof(T) codes per word with the first code in
// the most significant nibble, decode by scale / 7; quantize and single-payload decode only, as in
// the reference (its fused reduce is 8-bit).
//
// Mapping: as in the portable-format kernels, one lane owns 16 bytes of the tensor (4 fp32 or
// 8 half elements), a group sits in adjacent lanes of one DPP row, and every tile's loads are
// issued before the arithmetic.  Group strides of 66 or 68 bytes leave code words only 2- or
// 4-byte aligned; gfx950 global memory instructions accept that, so all accesses here are typed
// with element alignment only and there is no separate path for unaligned tensors.
#include "device_utils.h"
#include "launch.h"
#include "wire_common.h"

// Chunk size (log2 of the element count) from which the gather hop of interleaved 16-bit payloads stores group pairs
// as shifted dwords; below it the misaligned 8-byte stores measured faster (see wire_ring_step_kernel).
#ifndef LBC_PAIR_STORE_MIN_LOG2
#define LBC_PAIR_STORE_MIN_LOG2 22
#endif


namespace lbc {
namespace {

// ---------------------------------------------------------------------------
// quantize + pack (optionally x + residual), `world` chunks via blockIdx.y
// ---------------------------------------------------------------------------
template <typename T, int G, int BIT, bool HAS_R, bool COMPACT, int NT>
__global__ __launch_bounds__(kBlock) void wire_quant_kernel(const WireQuantArgs a) {
    constexpr int PNT = COMPACT ? kPlain : NT;
    using W = wire<T, BIT>;
    constexpr int VEC = W::VEC;
    constexpr int LPG = G / VEC;
    constexpr int UNROLL = 4;
    constexpr int BLOCK_ELEMS = W::TILE * kWavesPerBlock * UNROLL;
    static_assert(LPG >= 1 && LPG <= 16, "a group must fit one DPP row");

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t chunk = blockIdx.y;
    const int64_t chunk_start = chunk * a.shard_numel;
    int64_t valid = a.numel - chunk_start;
    valid = valid < 0 ? 0 : (valid > a.shard_numel ? a.shard_numel : valid);
    const int64_t groups = (a.shard_numel + G - 1) / G;
    const int64_t padded = groups * G;
    const group_layout<T, G, COMPACT, BIT> at{groups};
    // The reference sends a chunk of whole groups without a residual to its general kernels, whose running
    // maximum a NaN resets, and everything else to the fused pack kernel, whose fmaxf skips NaNs
    // (quant_pack_kernel.cu:231,259-262).
    const bool resets = !HAS_R && a.nan_resets != 0 && valid % G == 0;

    const T *__restrict__ x = static_cast<const T *>(a.x) + chunk_start;
    const T *__restrict__ r = HAS_R ? static_cast<const T *>(a.residual) + chunk_start : nullptr;
    uint8_t *__restrict__ payload = a.payloads + chunk * a.payload_stride;

    const int64_t block_first = static_cast<int64_t>(xcd_contiguous_block(BLOCK_ELEMS)) * BLOCK_ELEMS;
    if (block_first >= padded) return;

    using Raw = typename raw_bits<T>::type;
    auto multiplier_of = [&](float absmax) {
        const float scale = absmax < 1.0e-6f ? 1.0e-6f : absmax;   // a NaN stays and zeroes every code
        return W::LEVELS / scale;
    };
    auto group_multiplier = [&](uint32_t absmax_bits, float &absmax) {
        absmax = as_f32(group_max_bits<LPG>(absmax_bits));
        return multiplier_of(absmax);
    };
    // The scale of the lane's group as the reference's general kernels compute it, from the elements as stored.
    auto scan_scale = [&](const T (&elements)[VEC], int64_t group, int k0) {
        uint32_t mag[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) mag[i] = __builtin_bit_cast(Raw, elements[i]) & raw_bits<T>::ABS;
        return running_max_raw<T, G, VEC>(mag, k0, scan_start<T, G>(group));
    };
    auto clamp_codes = [&](int (&c)[VEC]) {
        constexpr int L = static_cast<int>(W::LEVELS);
#pragma unroll
        for (int i = 0; i < VEC; ++i) c[i] = c[i] < -L ? -L : (c[i] > L ? L : c[i]);
    };

    if (block_first + BLOCK_ELEMS <= valid) {
        T xv[UNROLL][VEC];
        T rv[UNROLL][VEC];
        int64_t e0[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            e0[u] = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * W::TILE + lane * VEC;
            load_elems<T, VEC, NT>(x + e0[u], xv[u]);
            if constexpr (HAS_R) load_elems<T, VEC, NT>(r + e0[u], rv[u]);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            float p[VEC];
            uint32_t m = 0;   // largest magnitude pattern; above the pattern of infinity when the lane holds a NaN
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                float v = widen(xv[u][i]);
                if constexpr (HAS_R) v = round_through<T>(v + widen(rv[u][i]));
                p[i] = v;
                const uint32_t bits = as_u32(v) & 0x7FFFFFFFu;
                m = bits > m ? bits : m;
            }
            const int64_t group = e0[u] / G;
            const int k0 = static_cast<int>(e0[u] - group * G);
            float absmax;
            float multiplier = group_multiplier(m, absmax);
            Raw stored = __builtin_bit_cast(Raw, narrow<T>(absmax));
            bool wide_codes = false;   // wavefront-uniform: codes may leave [-LEVELS, LEVELS]
            if (__ballot(m > 0x7F800000u) != 0) {   // a NaN somewhere in the wavefront: rare, and uniform
                if (!HAS_R && resets) {
                    const uint32_t scale_raw = scan_scale(xv[u], group, k0);
                    multiplier = multiplier_of(value_of<T>(scale_raw));
                    stored = static_cast<Raw>(scale_raw);
                    wide_codes = true;
                } else {                            // fmaxf skips NaNs
                    uint32_t skipping = 0;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) {
                        const uint32_t bits = as_u32(p[i]) & 0x7FFFFFFFu;
                        skipping = (bits <= 0x7F800000u && bits > skipping) ? bits : skipping;
                    }
                    multiplier = group_multiplier(skipping, absmax);
                    stored = __builtin_bit_cast(Raw, narrow<T>(absmax));
                }
            }
            int c[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) c[i] = cvt_i32(__builtin_rintf(p[i] * multiplier));
            if (wide_codes) clamp_codes(c);
            uint32_t words[W::WORDS];
            pack_codes<T, BIT, VEC, W::WORDS>(c, words);
            // Interleaved 16-bit payloads leave as misaligned 8-byte stores here.  Re-slicing a pair of 66-byte groups
            // into aligned dwords across lanes (store_group_pair16, what the ring's gather hop does) measured slower in
            // this kernel at every size, with operands rotated through 700 MB: 26.2 M bf16 elements 15.8 us as it is,
            // 17.7 us with non-temporal pair stores, 16.1 us with cached ones; 52.4 M 27.4 / 32.8 / 27.6 us.  Nor does
            // it pay to stage a wavefront's run of eight groups (528 bytes, 16-byte aligned) in LDS and carry it out
            // as 33 aligned 16-byte stores: 16.2 us (16.4 us non-temporal) against 15.6 us on 26.2 M elements, no
            // workgroup barrier involved.  The misaligned stores are not what this layout costs.
            store_piece<T, BIT, PNT, W::WORDS>(payload + at.codes(group) + piece_offset<T, BIT>(k0), words);
            if ((lane & (LPG - 1)) == 0) *reinterpret_cast<Raw *>(payload + at.scale(group)) = stored;
        }
        return;
    }

    // ---- edge block: ragged tail and zero padding, element-wise ----------------
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t e0 = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * W::TILE + lane * VEC;
        if (e0 - lane * VEC >= padded) break;  // wavefront-uniform
        float p[VEC];
        T held[VEC];
        uint32_t m = 0;
        bool has_nan = false;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            float v = 0.0f;
            held[i] = narrow<T>(0.0f);
            if (e < valid) {
                held[i] = x[e];
                v = widen(x[e]);
                if constexpr (HAS_R) v = round_through<T>(v + widen(r[e]));
            }
            p[i] = v;
            uint32_t bits = as_u32(v) & 0x7FFFFFFFu;
            has_nan |= bits > 0x7F800000u;
            bits = bits > 0x7F800000u ? 0u : bits;
            m = bits > m ? bits : m;
        }
        const int64_t group = e0 / G;
        const int k0 = static_cast<int>(e0 - group * G);
        float absmax;
        float multiplier = group_multiplier(m, absmax);   // every lane of the row takes part
        Raw stored = __builtin_bit_cast(Raw, narrow<T>(absmax));
        bool wide_codes = false;
        if constexpr (!HAS_R) {
            if (resets && __ballot(has_nan) != 0) {
                const uint32_t scale_raw = scan_scale(held, group, k0);
                multiplier = multiplier_of(value_of<T>(scale_raw));
                stored = static_cast<Raw>(scale_raw);
                wide_codes = true;
            }
        }
        if (e0 < padded) {   // the lane's VEC elements lie inside the padded range together: whole words again
            int c[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) c[i] = cvt_i32(__builtin_rintf(p[i] * multiplier));
            if (wide_codes) clamp_codes(c);
            uint32_t words[W::WORDS];
            pack_codes<T, BIT, VEC, W::WORDS>(c, words);
            store_piece<T, BIT, kPlain, W::WORDS>(payload + at.codes(group) + piece_offset<T, BIT>(k0), words);
            if ((lane & (LPG - 1)) == 0) *reinterpret_cast<Raw *>(payload + at.scale(group)) = stored;
        }
    }
}

template <typename T, int G, int BIT, bool HAS_R, bool COMPACT>
hipError_t launch_wire_quant_c(int mode, const WireQuantArgs &a, int world, hipStream_t stream) {
    constexpr int BLOCK_ELEMS = wire<T, BIT>::TILE * kWavesPerBlock * 4;
    const int64_t groups = (a.shard_numel + G - 1) / G;
    const int64_t blocks = (groups * G + BLOCK_ELEMS - 1) / BLOCK_ELEMS;
    if (blocks == 0 || world == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL || world > 65535) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(world));
    if (mode == kStream) hipLaunchKernelGGL((wire_quant_kernel<T, G, BIT, HAS_R, COMPACT, kNonTemporal>), grid, dim3(kBlock), 0, stream, a);
    else hipLaunchKernelGGL((wire_quant_kernel<T, G, BIT, HAS_R, COMPACT, kPlain>), grid, dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

template <typename T, int G, int BIT>
hipError_t launch_wire_quant_b(int mode, const WireQuantArgs &a, int world, hipStream_t stream) {
    if (a.residual != nullptr)
        return a.compact ? launch_wire_quant_c<T, G, BIT, true, true>(mode, a, world, stream)
                         : launch_wire_quant_c<T, G, BIT, true, false>(mode, a, world, stream);
    return a.compact ? launch_wire_quant_c<T, G, BIT, false, true>(mode, a, world, stream)
                     : launch_wire_quant_c<T, G, BIT, false, false>(mode, a, world, stream);
}

template <typename T, int G>
hipError_t launch_wire_quant_g(int bit, int mode, const WireQuantArgs &a, int world, hipStream_t stream) {
    if (bit == 8) return launch_wire_quant_b<T, G, 8>(mode, a, world, stream);
    if (bit == 4) return launch_wire_quant_b<T, G, 4>(mode, a, world, stream);
    return hipErrorNotSupported;
}

template <typename T>
hipError_t launch_wire_quant_t(int g, int bit, int mode, const WireQuantArgs &a, int world, hipStream_t s) {
    switch (g) {
        case 64: return launch_wire_quant_g<T, 64>(bit, mode, a, world, s);
        case 32: return launch_wire_quant_g<T, 32>(bit, mode, a, world, s);
        case 16: return launch_wire_quant_g<T, 16>(bit, mode, a, world, s);
        default: return hipErrorNotSupported;
    }
}

// ---------------------------------------------------------------------------
// fused dequant-reduce of up to 8 payloads (+ mean, + error-feedback update)
// ---------------------------------------------------------------------------
template <typename T, int G, int WORLD, bool FMA, bool COMPACT, int NT, bool WINDOWS = false>
__global__ __launch_bounds__(kBlock) void wire_reduce_kernel(const WireReduceArgs a) {
    constexpr int PNT = payload_load_hint<COMPACT, NT, WORLD>();
    using W = wire<T>;
    constexpr int VEC = W::VEC;
    constexpr int UNROLL = WORLD <= 2 ? 2 : 1;
    constexpr int BLOCK_ELEMS = W::TILE * kWavesPerBlock * UNROLL;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t block_first = static_cast<int64_t>(xcd_contiguous_block(BLOCK_ELEMS)) * BLOCK_ELEMS;
    const int64_t groups = (a.numel + G - 1) / G;
    const group_layout<T, G, COMPACT> at{groups};
    T *__restrict__ out = static_cast<T *>(a.out);
    const T *prepared = static_cast<const T *>(a.prepared);  // may alias new_r
    T *new_r = static_cast<T *>(a.new_residual);

    auto accumulate = [](float acc, float code, float step) {
        if constexpr (FMA) return __builtin_fmaf(code, step, acc);
        else return acc + code * step;
    };

    if (block_first + BLOCK_ELEMS <= a.numel) {
        uint32_t words[UNROLL][WORLD][W::WORDS];
        T stored[UNROLL][WORLD];
        int64_t e0[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            e0[u] = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * W::TILE + lane * VEC;
            const int64_t group = e0[u] / G;
            const int k0 = static_cast<int>(e0[u] - group * G);
            const int64_t code_at = at.codes(group) + k0;
            const int64_t scale_at = at.scale(group);
            if constexpr (WINDOWS) {   // 16-bit compact payloads below 2 GiB: aligned windows, scales out of them
                static_assert(COMPACT && sizeof(T) == 2 && G == 64 && W::WORDS == 2, "66-byte groups of 8 lanes");
                const uint32_t payload_bytes = static_cast<uint32_t>(groups * (G + 2));
#pragma unroll
                for (int r = 0; r < WORLD; ++r) {
                    const uint32_t lead = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(a.payloads[r]) & 3u);
                    uint32_t after;
                    load_piece16<window_policy<NT, WORLD>()>(buffer_over(a.payloads[r] - lead, window_span(payload_bytes + lead)),
                                          static_cast<uint32_t>(code_at) + lead, words[u][r], after);
                    const uint32_t raw = from_last_lane_of_8(after, (lane & 8) != 0);
                    stored[u][r] = __builtin_bit_cast(T, static_cast<uint16_t>(raw));
                }
            } else {
#pragma unroll
                for (int r = 0; r < WORLD; ++r) {
                    load_words<W::WORDS, sizeof(T), PNT>(a.payloads[r] + code_at, words[u][r]);
                    stored[u][r] = *reinterpret_cast<const T *>(a.payloads[r] + scale_at);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            float acc[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
#pragma unroll
            for (int r = 0; r < WORLD; ++r) {
                const float step = div127(widen(stored[u][r]));
#pragma unroll
                for (int i = 0; i < VEC; ++i)
                    acc[i] = accumulate(acc[i], code_to_float(words[u][r][i / 4], byte_in_word<T>(i % 4)), step);
            }
            T o[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                acc[i] = acc[i] * a.inv_divisor;
                o[i] = narrow<T>(acc[i]);
            }
            store_elems<T, VEC, NT>(out + e0[u], o);
            if (new_r != nullptr) {
                T pv[VEC], d[VEC];
                load_elems<T, VEC, NT>(prepared + e0[u], pv);
#pragma unroll
                for (int i = 0; i < VEC; ++i) d[i] = narrow<T>(widen(pv[i]) - acc[i]);
                store_elems<T, VEC, NT>(new_r + e0[u], d);
            }
        }
        return;
    }

    for (int u = 0; u < UNROLL; ++u) {
        const int64_t e0 = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * W::TILE + lane * VEC;
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            if (e >= a.numel) break;
            const int64_t group = e / G;
            const int k = static_cast<int>(e - group * G);
            float acc = 0.0f;
#pragma unroll
            for (int r = 0; r < WORLD; ++r) {
                const float step = div127(widen(*reinterpret_cast<const T *>(a.payloads[r] + at.scale(group))));
                const float code = static_cast<float>(static_cast<int8_t>(a.payloads[r][at.codes(group) + byte_in_group<T>(k)]));
                acc = accumulate(acc, code, step);
            }
            acc = acc * a.inv_divisor;
            out[e] = narrow<T>(acc);
            if (new_r != nullptr) new_r[e] = narrow<T>(widen(prepared[e]) - acc);
        }
    }
}

template <typename T, int G, int WORLD, bool FMA, bool COMPACT>
hipError_t launch_wire_reduce_c(int mode, const WireReduceArgs &a, hipStream_t stream) {
    constexpr int BLOCK_ELEMS = wire<T>::TILE * kWavesPerBlock * (WORLD <= 2 ? 2 : 1);
    const int64_t blocks = (a.numel + BLOCK_ELEMS - 1) / BLOCK_ELEMS;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks));
    if constexpr (COMPACT && sizeof(T) == 2) {
        if ((a.numel + G - 1) / G * (G + 2) < (1LL << 31)) {   // a buffer descriptor spans the payload
            if (mode == kStream) hipLaunchKernelGGL((wire_reduce_kernel<T, G, WORLD, FMA, COMPACT, kNonTemporal, true>), grid, dim3(kBlock), 0, stream, a);
            else hipLaunchKernelGGL((wire_reduce_kernel<T, G, WORLD, FMA, COMPACT, kPlain, true>), grid, dim3(kBlock), 0, stream, a);
            return hipGetLastError();
        }
    }
    if (mode == kStream) hipLaunchKernelGGL((wire_reduce_kernel<T, G, WORLD, FMA, COMPACT, kNonTemporal>), grid, dim3(kBlock), 0, stream, a);
    else hipLaunchKernelGGL((wire_reduce_kernel<T, G, WORLD, FMA, COMPACT, kPlain>), grid, dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

template <typename T, int G, int WORLD, bool FMA>
hipError_t launch_wire_reduce_w(int mode, const WireReduceArgs &a, hipStream_t stream) {
    return a.compact ? launch_wire_reduce_c<T, G, WORLD, FMA, true>(mode, a, stream)
                     : launch_wire_reduce_c<T, G, WORLD, FMA, false>(mode, a, stream);
}

template <typename T, int G, bool FMA>
hipError_t launch_wire_reduce_f(int world, int mode, const WireReduceArgs &a, hipStream_t s) {
    switch (world) {
        case 1: return launch_wire_reduce_w<T, G, 1, FMA>(mode, a, s);
        case 2: return launch_wire_reduce_w<T, G, 2, FMA>(mode, a, s);
        case 3: return launch_wire_reduce_w<T, G, 3, FMA>(mode, a, s);
        case 4: return launch_wire_reduce_w<T, G, 4, FMA>(mode, a, s);
        case 5: return launch_wire_reduce_w<T, G, 5, FMA>(mode, a, s);
        case 6: return launch_wire_reduce_w<T, G, 6, FMA>(mode, a, s);
        case 7: return launch_wire_reduce_w<T, G, 7, FMA>(mode, a, s);
        case 8: return launch_wire_reduce_w<T, G, 8, FMA>(mode, a, s);
        default: return hipErrorNotSupported;
    }
}

template <typename T>
hipError_t launch_wire_reduce_t(int g, int world, bool fma, int mode, const WireReduceArgs &a, hipStream_t s) {
    if (g != 64) return hipErrorNotSupported;   // as the reference: dequant_reduce_kernel.cu:17,252
    return fma ? launch_wire_reduce_f<T, 64, true>(world, mode, a, s) : launch_wire_reduce_f<T, 64, false>(world, mode, a, s);
}

// ---------------------------------------------------------------------------
// decode of one payload (optionally combined into `out`), or of `world` shard payloads
// ---------------------------------------------------------------------------
template <typename T, int OP> __device__ __forceinline__ float combine_in(float old, float v) {
    if constexpr (OP == 1) return add_in<T>(old, v);
    else if constexpr (OP == 2) return old > v ? old : v;
    else if constexpr (OP == 3) return old > v ? v : old;
    else return v;
}

template <typename T, int G, int BIT, int OP, bool COMPACT, int NT>
__global__ __launch_bounds__(kBlock) void wire_decode_kernel(const WireDecodeArgs a) {
    constexpr int PNT = payload_load_hint<COMPACT, NT, 1>();
    using W = wire<T, BIT>;
    constexpr int VEC = W::VEC;
    constexpr int UNROLL = 2;
    constexpr int BLOCK_ELEMS = W::TILE * kWavesPerBlock * UNROLL;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t chunk = blockIdx.y;
    const int64_t chunk_start = chunk * a.shard_numel;
    int64_t valid = a.total_numel - chunk_start;
    valid = valid < 0 ? 0 : (valid > a.shard_numel ? a.shard_numel : valid);
    const int64_t groups = (a.shard_numel + G - 1) / G;
    const group_layout<T, G, COMPACT, BIT> at{groups};
    const uint8_t *__restrict__ payload = a.payloads + chunk * a.payload_stride;
    T *__restrict__ out = static_cast<T *>(a.out) + chunk_start;
    const int64_t block_first = static_cast<int64_t>(xcd_contiguous_block(BLOCK_ELEMS)) * BLOCK_ELEMS;
    if (block_first >= valid) return;

    if (block_first + BLOCK_ELEMS <= valid) {
        uint32_t words[UNROLL][W::WORDS];
        T stored[UNROLL];
        int64_t e0[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            e0[u] = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * W::TILE + lane * VEC;
            const int64_t group = e0[u] / G;
            const int k0 = static_cast<int>(e0[u] - group * G);
            load_piece<T, BIT, PNT, W::WORDS>(payload + at.codes(group) + piece_offset<T, BIT>(k0), words[u]);
            stored[u] = *reinterpret_cast<const T *>(payload + at.scale(group));
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            T o[VEC];
            if constexpr (OP != 0) load_elems<T, VEC, NT>(out + e0[u], o);
            const float step = step_of<BIT>(widen(stored[u]));
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                float v = round_through<T>(unpack_code<T, BIT, W::WORDS>(words[u], i) * step);
                if constexpr (OP != 0) v = combine_in<T, OP>(widen(o[i]), v);
                o[i] = narrow<T>(v);
            }
            store_elems<T, VEC, NT>(out + e0[u], o);
        }
        return;
    }

    for (int u = 0; u < UNROLL; ++u) {
        const int64_t e0 = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * W::TILE + lane * VEC;
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            if (e >= valid) break;
            const int64_t group = e / G;
            const int k = static_cast<int>(e - group * G);
            const float step = step_of<BIT>(widen(*reinterpret_cast<const T *>(payload + at.scale(group))));
            float v = round_through<T>(code_at<T, BIT>(payload + at.codes(group), k) * step);
            if constexpr (OP != 0) v = combine_in<T, OP>(widen(out[e]), v);
            out[e] = narrow<T>(v);
        }
    }
}

template <typename T, int G, int BIT, int OP, bool COMPACT>
hipError_t launch_wire_decode_c(int mode, const WireDecodeArgs &a, int world, hipStream_t stream) {
    constexpr int BLOCK_ELEMS = wire<T, BIT>::TILE * kWavesPerBlock * 2;
    const int64_t blocks = (a.shard_numel + BLOCK_ELEMS - 1) / BLOCK_ELEMS;
    if (blocks == 0 || world == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL || world > 65535) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(world));
    if (mode == kStream) hipLaunchKernelGGL((wire_decode_kernel<T, G, BIT, OP, COMPACT, kNonTemporal>), grid, dim3(kBlock), 0, stream, a);
    else hipLaunchKernelGGL((wire_decode_kernel<T, G, BIT, OP, COMPACT, kPlain>), grid, dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

template <typename T, int G, int BIT, int OP>
hipError_t launch_wire_decode_op(int mode, const WireDecodeArgs &a, int world, hipStream_t stream) {
    return a.compact ? launch_wire_decode_c<T, G, BIT, OP, true>(mode, a, world, stream)
                     : launch_wire_decode_c<T, G, BIT, OP, false>(mode, a, world, stream);
}

template <typename T, int G, int BIT>
hipError_t launch_wire_decode_b(int op, int mode, const WireDecodeArgs &a, int world, hipStream_t s) {
    switch (op) {
        case 0: return launch_wire_decode_op<T, G, BIT, 0>(mode, a, world, s);
        case 1: return launch_wire_decode_op<T, G, BIT, 1>(mode, a, world, s);
        case 2: return launch_wire_decode_op<T, G, BIT, 2>(mode, a, world, s);
        case 3: return launch_wire_decode_op<T, G, BIT, 3>(mode, a, world, s);
        default: return hipErrorNotSupported;
    }
}

template <typename T, int G>
hipError_t launch_wire_decode_g(int bit, int op, int mode, const WireDecodeArgs &a, int world, hipStream_t s) {
    if (bit == 8) return launch_wire_decode_b<T, G, 8>(op, mode, a, world, s);
    if (bit == 4) return launch_wire_decode_b<T, G, 4>(op, mode, a, world, s);
    return hipErrorNotSupported;
}

template <typename T>
hipError_t launch_wire_decode_t(int g, int bit, int op, int mode, const WireDecodeArgs &a, int world, hipStream_t s) {
    switch (g) {
        case 64: return launch_wire_decode_g<T, 64>(bit, op, mode, a, world, s);
        case 32: return launch_wire_decode_g<T, 32>(bit, op, mode, a, world, s);
        case 16: return launch_wire_decode_g<T, 16>(bit, op, mode, a, world, s);
        default: return hipErrorNotSupported;
    }
}

// ---------------------------------------------------------------------------
// ring / tree step in this format: chunk (op)= decode(received) [* 1/W], then the quantize of the updated chunk
// ---------------------------------------------------------------------------
// What a rank running the reference does per hop with its extension loaded (torch_topology.py:262-316): decode the
// arriving payload into the chunk with reduce op SUM or NONE, `div_` by the world size on the hop that completes
// the sum (a multiplication by the float reciprocal, the way torch divides a device tensor by a number), then
// quantize the chunk for the next hop - here in one launch, the updated chunk still in registers.  Linear 8-bit
// codes, whole groups (the reference's in-place decode needs them).  The encode is the one a chunk of whole groups
// without a residual gets in the reference: group maximum with NaNs skipped, and when a group holds a NaN the
// running maximum of the general kernels, which a NaN resets (see wire_quant_kernel).
template <typename T, bool ACC> constexpr int wire_ring_unroll() { return ACC || sizeof(T) == 2 ? 1 : 4; }

template <typename T, int G, bool COMPACT, int NT, bool ACC, bool WINDOWS = false>
__global__ __launch_bounds__(kBlock) void wire_ring_step_kernel(const WireRingStepArgs a) {
    constexpr int PNT_LOAD = payload_load_hint<COMPACT, NT, 1>();
    constexpr int PNT_STORE = COMPACT ? kPlain : NT;
    using W = wire<T, 8>;
    using Raw = typename raw_bits<T>::type;
    constexpr int VEC = W::VEC;
    constexpr int LPG = G / VEC;
    // Tiles in flight per wavefront, as measured on 6.5 M to 52 M element chunks: one for the accumulating step and
    // for 16-bit chunks, four for the write-only steps on fp32 chunks.
    constexpr int UNROLL = wire_ring_unroll<T, ACC>();
    constexpr int BLOCK_ELEMS = W::TILE * kWavesPerBlock * UNROLL;
    static_assert(LPG >= 1 && LPG <= 16, "a group must fit one DPP row");

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t groups = a.numel / G;               // whole groups only
    const group_layout<T, G, COMPACT, 8> at{groups};
    const uint8_t *__restrict__ received = a.received;
    T *chunk = static_cast<T *>(a.chunk);
    const bool scaled = a.inv_divisor != 1.0f;
    const bool emit = a.send != nullptr;
    const int64_t block_first = static_cast<int64_t>(xcd_contiguous_block(BLOCK_ELEMS)) * BLOCK_ELEMS;
    if (block_first >= a.numel) return;

    uint32_t words[UNROLL][W::WORDS];
    T stored[UNROLL];
    T xv[UNROLL][VEC];
    int64_t e0[UNROLL];
    bool live[UNROLL];   // a lane's elements, and its whole group, lie inside the chunk or outside it together
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        e0[u] = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * W::TILE + lane * VEC;
        live[u] = e0[u] < a.numel;
        if constexpr (WINDOWS) {   // 16-bit compact payload below 2 GiB: aligned windows, the scale out of them;
            static_assert(COMPACT && sizeof(T) == 2 && G == 64 && W::WORDS == 2, "66-byte groups of 8 lanes");
            const int64_t group = e0[u] / G;                    // a window past the payload reads as zeros
            const int k0 = static_cast<int>(e0[u] - group * G);
            const uint32_t lead = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(received) & 3u);
            uint32_t after;
            load_piece16<window_policy<NT, 1>()>(buffer_over(received - lead, window_span(static_cast<uint32_t>(groups * (G + 2)) + lead)),
                                                 static_cast<uint32_t>(live[u] ? at.codes(group) + k0 : 0) + lead, words[u], after);
            stored[u] = __builtin_bit_cast(T, static_cast<uint16_t>(from_last_lane_of_8(after, (lane & 8) != 0)));
            if constexpr (ACC) {
                if (live[u]) load_elems<T, VEC, NT>(chunk + e0[u], xv[u]);
            }
        } else if (live[u]) {
            const int64_t group = e0[u] / G;
            const int k0 = static_cast<int>(e0[u] - group * G);
            load_piece<T, 8, PNT_LOAD, W::WORDS>(received + at.codes(group) + piece_offset<T, 8>(k0), words[u]);
            stored[u] = *reinterpret_cast<const T *>(received + at.scale(group));
            if constexpr (ACC) load_elems<T, VEC, NT>(chunk + e0[u], xv[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        float p[VEC];
        T held[VEC];
        uint32_t m = 0;   // largest magnitude pattern; above the pattern of infinity when the lane holds a NaN
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            p[i] = 0.0f;
            held[i] = narrow<T>(0.0f);
        }
        if (live[u]) {
            const float step = step_of<8>(widen(stored[u]));
#pragma unroll
            for (int i = 0; i < VEC; ++i) p[i] = unpack_code<T, 8, W::WORDS>(words[u], i) * step;
            round_through_all<T, VEC>(p);
            if constexpr (ACC) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) p[i] = widen(xv[u][i]) + p[i];
                round_through_all<T, VEC>(p);
            }
            if (scaled) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) p[i] = p[i] * a.inv_divisor;
                round_through_all<T, VEC>(p);
            }
            narrow_all<T, VEC>(p, held);
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                const uint32_t bits = as_u32(p[i]) & 0x7FFFFFFFu;
                m = bits > m ? bits : m;
            }
            store_elems<T, VEC, NT>(chunk + e0[u], held);
        }
        if (!emit) continue;    // uniform over the grid
        // every lane of a row takes part in the group reductions; rows past the end carry zeros
        const int64_t group = e0[u] / G;
        const int k0 = static_cast<int>(e0[u] - group * G);
        const float absmax = as_f32(group_max_bits<LPG>(m));   // the group maximum when the wavefront holds no NaN
        float scale = absmax < 1.0e-6f ? 1.0e-6f : absmax;
        Raw kept = __builtin_bit_cast(Raw, narrow<T>(absmax));
        bool wide_codes = false;                               // wavefront-uniform
        if (__ballot(m > 0x7F800000u) != 0) {                  // a NaN somewhere: every group is scanned again
            uint32_t mag[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) mag[i] = __builtin_bit_cast(Raw, held[i]) & raw_bits<T>::ABS;
            const uint32_t scale_raw = running_max_raw<T, G, VEC>(mag, k0, scan_start<T, G>(group));
            const float rescanned = value_of<T>(scale_raw);
            scale = rescanned < 1.0e-6f ? 1.0e-6f : rescanned;
            kept = static_cast<Raw>(scale_raw);
            wide_codes = true;
        }
        const float multiplier = W::LEVELS / scale;
        int c[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            c[i] = cvt_i32(__builtin_rintf(p[i] * multiplier));
            if (wide_codes) c[i] = c[i] < -127 ? -127 : (c[i] > 127 ? 127 : c[i]);
        }
        uint32_t out_words[W::WORDS];
        pack_codes<T, 8, VEC, W::WORDS>(c, out_words);
        if constexpr (WINDOWS) {
            // The hop that only decodes and requantizes, from 4 Mi elements on (uniform): the payload leaves as
            // whole dwords shifted across lanes, with the non-temporal hint.  Measured with operands rotated through
            // 700 MB, bf16: 52 M elements 38.8 instead of 43.3 us, 26 M 19.8 instead of 21.5, 13.1 M 11.4 instead
            // of 12.9, 6.5 M 7.3 instead of 8.3; 3.3 M 6.3 against 5.3 and 1.6 M 4.5 either way, hence the bound.
            // (With only a few buffer sets, i.e. payloads that stay in the last-level cache, 13.1 M read 11.4
            // against 10.9 us, which is where an earlier bound of 16 Mi came from.)  Both forms write exactly the
            // chunk and the payload (rocprofv3 WRITE_SIZE 38,800 KiB against 39,082 KiB on 13.1 M elements) and read
            // exactly the payload: the gain is in the store instructions, not in traffic.  The accumulating hop and
            // the quantize kernel lost 1-20 % with the same stores.
            if ((reinterpret_cast<uintptr_t>(a.send) & 3u) == 0 && a.numel >= (int64_t{1} << LBC_PAIR_STORE_MIN_LOG2)) {
                store_group_pair16<kNonTemporal>(a.send + at.codes(group & ~int64_t{1}), lane, out_words, kept, live[u],
                                              (group | 1) < groups);
                continue;
            }
        }
        if (!live[u]) continue;
        store_piece<T, 8, PNT_STORE, W::WORDS>(a.send + at.codes(group) + piece_offset<T, 8>(k0), out_words);
        if ((lane & (LPG - 1)) == 0) *reinterpret_cast<Raw *>(a.send + at.scale(group)) = kept;
    }
}

template <typename T, int G, bool COMPACT, bool ACC>
hipError_t launch_wire_ring_c(int mode, const WireRingStepArgs &a, hipStream_t stream) {
    constexpr int BLOCK_ELEMS = wire<T, 8>::TILE * kWavesPerBlock * wire_ring_unroll<T, ACC>();
    const int64_t blocks = (a.numel + BLOCK_ELEMS - 1) / BLOCK_ELEMS;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks));
    // Aligned windows for the received payload pay on the hop that only decodes and requantizes (52 M bf16
    // elements: 43 against 47.5 us); on the accumulating hop, where the chunk is read as well, they measured 2 %
    // slower, and a single-payload decode does not notice them (the payload is a third of its traffic).
    if constexpr (COMPACT && sizeof(T) == 2 && G == 64 && !ACC) {
        if (a.numel / G * (G + 2) < (1LL << 31)) {   // a buffer descriptor spans the payload
            if (mode == kStream) hipLaunchKernelGGL((wire_ring_step_kernel<T, G, COMPACT, kNonTemporal, ACC, true>), grid, dim3(kBlock), 0, stream, a);
            else hipLaunchKernelGGL((wire_ring_step_kernel<T, G, COMPACT, kPlain, ACC, true>), grid, dim3(kBlock), 0, stream, a);
            return hipGetLastError();
        }
    }
    if (mode == kStream) hipLaunchKernelGGL((wire_ring_step_kernel<T, G, COMPACT, kNonTemporal, ACC>), grid, dim3(kBlock), 0, stream, a);
    else hipLaunchKernelGGL((wire_ring_step_kernel<T, G, COMPACT, kPlain, ACC>), grid, dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

template <typename T, int G>
hipError_t launch_wire_ring_g(bool accumulate, int mode, const WireRingStepArgs &a, hipStream_t s) {
    if (a.compact) return accumulate ? launch_wire_ring_c<T, G, true, true>(mode, a, s) : launch_wire_ring_c<T, G, true, false>(mode, a, s);
    return accumulate ? launch_wire_ring_c<T, G, false, true>(mode, a, s) : launch_wire_ring_c<T, G, false, false>(mode, a, s);
}

template <typename T>
hipError_t launch_wire_ring_t(int g, bool accumulate, int mode, const WireRingStepArgs &a, hipStream_t s) {
    switch (g) {
        case 64: return launch_wire_ring_g<T, 64>(accumulate, mode, a, s);
        case 32: return launch_wire_ring_g<T, 32>(accumulate, mode, a, s);
        case 16: return launch_wire_ring_g<T, 16>(accumulate, mode, a, s);
        default: return hipErrorNotSupported;
    }
}

}  // namespace

hipError_t launch_wire_quant(int dtype, int group_size, int bit, int mode, const WireQuantArgs &args, int world,
                             hipStream_t stream) {
    switch (dtype) {
        case kF32: return launch_wire_quant_t<float>(group_size, bit, mode, args, world, stream);
        case kF16: return launch_wire_quant_t<f16>(group_size, bit, mode, args, world, stream);
        case kBF16: return launch_wire_quant_t<bf16>(group_size, bit, mode, args, world, stream);
        default: return hipErrorNotSupported;
    }
}

hipError_t launch_wire_reduce(int dtype, int group_size, int world, bool fused_multiply_add, int mode,
                              const WireReduceArgs &args, hipStream_t stream) {
    switch (dtype) {
        case kF32: return launch_wire_reduce_t<float>(group_size, world, fused_multiply_add, mode, args, stream);
        case kF16: return launch_wire_reduce_t<f16>(group_size, world, fused_multiply_add, mode, args, stream);
        case kBF16: return launch_wire_reduce_t<bf16>(group_size, world, fused_multiply_add, mode, args, stream);
        default: return hipErrorNotSupported;
    }
}

hipError_t launch_wire_decode(int dtype, int group_size, int bit, int reduce_op, int mode, const WireDecodeArgs &args,
                              int world, hipStream_t stream) {
    switch (dtype) {
        case kF32: return launch_wire_decode_t<float>(group_size, bit, reduce_op, mode, args, world, stream);
        case kF16: return launch_wire_decode_t<f16>(group_size, bit, reduce_op, mode, args, world, stream);
        case kBF16: return launch_wire_decode_t<bf16>(group_size, bit, reduce_op, mode, args, world, stream);
        default: return hipErrorNotSupported;
    }
}

hipError_t launch_wire_ring_step(int dtype, int group_size, bool accumulate, int mode, const WireRingStepArgs &args,
                                 hipStream_t stream) {
    switch (dtype) {
        case kF32: return launch_wire_ring_t<float>(group_size, accumulate, mode, args, stream);
        case kF16: return launch_wire_ring_t<f16>(group_size, accumulate, mode, args, stream);
        case kBF16: return launch_wire_ring_t<bf16>(group_size, accumulate, mode, args, stream);
        default: return hipErrorNotSupported;
    }
}

}  // namespace lbc
