// One compute step of the quantized ring all-reduce on one chunk of the bucket, for gfx950.
//
// The ring schedule of the reference (ccdl_comm/cuda/transports/pipelined_ring.py:216-275) alternates, on every
// rank, "decode the payload that arrived into chunk c of the bucket" with "quantize chunk c and send it on":
// the chunk a step reduces into is always the chunk the next step sends.  The reference runs these as two
// kernels (ccdl_comm/cuda/transports/torch_topology.py:236-316: dequantize with reduce_op sum or none, an in-place
// division at the last reduce step, then quantize), which reads the chunk twice and writes it once.  Here the
// updated chunk is quantized while it is still in registers: one launch reads the received payload and the
// chunk, writes the chunk and the next payload.
//
// Per element, in the order the two-kernel sequence rounds:
//   d = T(float(code) * scale)                  decode, rounded to the chunk's type T
//   v = T(float(chunk) + d)      (ACC only)     the in-place sum in T arithmetic
//   v = T(v / divisor)           (divisor != 1) the in-place mean (divide_all)
//   chunk = v;  payload = quantize(v)           same group maximum, scale and rounding as quant_pack_kernel
//
// Mapping: one lane owns 16 bytes of the chunk (4 fp32 or 8 16-bit elements), a group sits in adjacent lanes of
// one DPP row, a 256-thread block walks UNROLL * 4 wavefront tiles with every load issued before the first use.
#include "device_utils.h"
#include "launch.h"

namespace lbc {
namespace {

// Tiles in flight per wavefront, as measured on 1.6 M to 26 M element chunks: the accumulating step, which reads
// and writes the chunk, is fastest with one (more wavefronts resident), the write-only steps with four (fp32) or
// two (16-bit) tiles of loads issued ahead.
template <typename T, bool ACC> struct ring_tiling {
    static constexpr int VEC = 16 / sizeof(T);
    static constexpr int TILE = kWave * VEC;
    static constexpr int UNROLL = ACC ? 1 : (sizeof(T) == 4 ? 4 : 2);
    static constexpr int BLOCK_ELEMS = TILE * kWavesPerBlock * UNROLL;
};

template <typename T, int G, int MODE, bool ACC>
__global__ __launch_bounds__(kBlock) void ring_step_kernel(const RingStepArgs a) {
    using L = ring_tiling<T, ACC>;
    constexpr int VEC = L::VEC;
    constexpr int LPG = G / VEC;
    constexpr int UNROLL = L::UNROLL;
    // The one code stream is a fifth of the traffic at most; without the non-temporal hint it measures faster, as in
    // the single-payload decode kernel.
    constexpr int kCodeLoad = MODE == kStream ? kVector : MODE;
    static_assert(LPG >= 1 && LPG <= 16, "a group must fit one DPP row");

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t padded = (a.numel + G - 1) / G * G;
    const int64_t block_first = static_cast<int64_t>(xcd_contiguous_block(L::BLOCK_ELEMS)) * L::BLOCK_ELEMS;
    if (block_first >= padded) return;

    T *chunk = static_cast<T *>(a.chunk);  // read and written by the same lane: no restrict
    const int8_t *__restrict__ recv_codes = a.recv_codes;
    const float *__restrict__ recv_scales = a.recv_scales;
    const bool mean = a.divisor != 1.0f;
    const bool emit = a.send_codes != nullptr;  // uniform over the grid

    if (MODE != kScalar && block_first + L::BLOCK_ELEMS <= a.numel) {
        // ---- interior block: every tile is full ----
        T xv[UNROLL][VEC];
        uint32_t words[UNROLL][VEC / 4];
        float rscale[UNROLL];
        int64_t e0[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            e0[u] = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * L::TILE + lane * VEC;
            load_vec<uint32_t, VEC / 4, kCodeLoad>(reinterpret_cast<const uint32_t *>(recv_codes + e0[u]), words[u]);
            rscale[u] = recv_scales[e0[u] / G];
            if constexpr (ACC) load_wide<T, VEC, MODE>(chunk + e0[u], xv[u]);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            float p[VEC];
            T out[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) p[i] = code_to_float(words[u][i / 4], i % 4) * rscale[u];
            round_through_all<T, VEC>(p);
            if constexpr (ACC) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) p[i] = widen(xv[u][i]) + p[i];
                round_through_all<T, VEC>(p);
            }
            if (mean) divide_all<T, VEC>(p, a.divisor);
            narrow_all<T, VEC>(p, out);
            store_wide<T, VEC, MODE>(chunk + e0[u], out);
            if (emit) {
                const float scale = group_scale<VEC, LPG>(p);
                int c[VEC];
                encode_group<VEC>(p, scale, c);
                uint32_t packed[VEC / 4];
#pragma unroll
                for (int k = 0; k < VEC / 4; ++k) packed[k] = pack4(c[4 * k], c[4 * k + 1], c[4 * k + 2], c[4 * k + 3]);
                store_vec<uint32_t, VEC / 4, MODE>(reinterpret_cast<uint32_t *>(a.send_codes + e0[u]), packed);
                if ((lane & (LPG - 1)) == 0) a.send_scales[e0[u] / G] = scale;
            }
        }
        return;
    }

    // ---- edge block: ragged tail and zero padding, element-wise and guarded ----
    for (int u = 0; u < UNROLL; ++u) {
        const int64_t e0 = block_first + static_cast<int64_t>(tile_in_block<UNROLL>(u, wave)) * L::TILE + lane * VEC;
        if (e0 - lane * VEC >= padded) continue;  // wavefront-uniform
        const float rscale = e0 < padded ? recv_scales[e0 / G] : 0.0f;
        float p[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const int64_t e = e0 + i;
            float v = 0.0f;
            if (e < a.numel) {
                v = round_through<T>(static_cast<float>(recv_codes[e]) * rscale);
                if constexpr (ACC) v = round_through<T>(widen(chunk[e]) + v);
                if (mean) v = round_through<T>(v / a.divisor);
                chunk[e] = narrow<T>(v);
            }
            p[i] = v;
        }
        if (emit) {
            // Every lane of the row takes part in the butterfly, also lanes past the padded end (zeros).
            const float scale = group_scale<VEC, LPG>(p);
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                const int64_t e = e0 + i;
                if (e < padded) a.send_codes[e] = static_cast<int8_t>(encode(p[i], scale));
            }
            if ((lane & (LPG - 1)) == 0 && e0 < padded) a.send_scales[e0 / G] = scale;
        }
    }
}

template <typename T, int G, bool ACC>
hipError_t launch_ring_g(int mode, const RingStepArgs &a, hipStream_t stream) {
    using L = ring_tiling<T, ACC>;
    const int64_t padded = (a.numel + G - 1) / G * G;
    const int64_t blocks = (padded + L::BLOCK_ELEMS - 1) / L::BLOCK_ELEMS;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    const dim3 grid(static_cast<unsigned>(blocks));
    switch (mode) {
        case kStream: hipLaunchKernelGGL((ring_step_kernel<T, G, kStream, ACC>), grid, dim3(kBlock), 0, stream, a); break;
        case kVector: hipLaunchKernelGGL((ring_step_kernel<T, G, kVector, ACC>), grid, dim3(kBlock), 0, stream, a); break;
        default: hipLaunchKernelGGL((ring_step_kernel<T, G, kScalar, ACC>), grid, dim3(kBlock), 0, stream, a); break;
    }
    return hipGetLastError();
}

template <typename T>
hipError_t launch_ring_t(int g, bool accumulate, int mode, const RingStepArgs &a, hipStream_t s) {
    switch (g) {
        case 64: return accumulate ? launch_ring_g<T, 64, true>(mode, a, s) : launch_ring_g<T, 64, false>(mode, a, s);
        case 32: return accumulate ? launch_ring_g<T, 32, true>(mode, a, s) : launch_ring_g<T, 32, false>(mode, a, s);
        case 16: return accumulate ? launch_ring_g<T, 16, true>(mode, a, s) : launch_ring_g<T, 16, false>(mode, a, s);
        default: return hipErrorNotSupported;
    }
}

}  // namespace

hipError_t launch_ring_step(int dtype, int group_size, bool accumulate, int mode, const RingStepArgs &args,
                            hipStream_t stream) {
    switch (dtype) {
        case kF32: return launch_ring_t<float>(group_size, accumulate, mode, args, stream);
        case kF16: return launch_ring_t<f16>(group_size, accumulate, mode, args, stream);
        case kBF16: return launch_ring_t<bf16>(group_size, accumulate, mode, args, stream);
        default: return hipErrorNotSupported;
    }
}

}  // namespace lbc
