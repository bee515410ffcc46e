// What a trivial streaming kernel reaches on this part: read-only, write-only, copy, a 16-bytes-in / 4-bytes-out
// kernel (the traffic shape of an fp32 quantize) and an 8 x 4-bytes-in (+ 8 scales) / 16-bytes-out kernel (the
// traffic shape of the W=8 fused reduce) over rotating buffers, one workgroup per tile or a grid-stride loop, with
// and without the non-temporal hint.  They do no arithmetic worth the name: the codec kernels are judged against
// these figures as well as against the 8 TB/s on the data sheet, and tests/test_zx_streaming_ceiling.py holds the hot
// kernels to 0.9 of the row with their traffic mix.
// Usage: stream_probe [MiB per buffer, default 100]           the table
//        stream_probe rows <elements of a W=8 reduce> <elements of an fp32 quantize> [<elements of a 16-bit quantize>]
//                                                             machine-readable rows: "ROW name microseconds bytes"
//        stream_probe depth                                   the plain kernels against the number of buffers in rotation
// Not part of the product.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
typedef float float4v __attribute__((ext_vector_type(4)));

template <int UNROLL, bool NT>
__global__ __launch_bounds__(256) void read_kernel(const float4v* __restrict__ in, float* __restrict__ out, size_t n4) {
    size_t base = (size_t)blockIdx.x * 256 * UNROLL + threadIdx.x;
    float4v acc = {0, 0, 0, 0};
    float4v v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        size_t i = base + (size_t)u * 256;
        if (i < n4) v[u] = NT ? __builtin_nontemporal_load(in + i) : in[i]; else v[u] = acc;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc += v[u];
    if (acc.x + acc.y + acc.z + acc.w == 12345.678f) out[0] = 1.0f;
}

template <int UNROLL, bool NT>
__global__ __launch_bounds__(256) void read_gs_kernel(const float4v* __restrict__ in, float* __restrict__ out, size_t n4) {
    // grid-stride persistent
    float4v acc = {0, 0, 0, 0};
    size_t stride = (size_t)gridDim.x * 256 * UNROLL;
    for (size_t base = (size_t)blockIdx.x * 256 * UNROLL + threadIdx.x; base < n4; base += stride) {
        float4v v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            size_t i = base + (size_t)u * 256;
            if (i < n4) v[u] = NT ? __builtin_nontemporal_load(in + i) : in[i]; else v[u] = float4v{0,0,0,0};
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc += v[u];
    }
    if (acc.x + acc.y + acc.z + acc.w == 12345.678f) out[0] = 1.0f;
}

template <int UNROLL, bool NT>
__global__ __launch_bounds__(256) void write_kernel(float4v* __restrict__ out, size_t n4) {
    size_t base = (size_t)blockIdx.x * 256 * UNROLL + threadIdx.x;
    float4v v = {1.0f, 2.0f, 3.0f, (float)threadIdx.x};
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        size_t i = base + (size_t)u * 256;
        if (i < n4) { if (NT) __builtin_nontemporal_store(v, out + i); else out[i] = v; }
    }
}

template <int UNROLL, bool NT>
__global__ __launch_bounds__(256) void copy_kernel(const float4v* __restrict__ in, float4v* __restrict__ out, size_t n4) {
    size_t base = (size_t)blockIdx.x * 256 * UNROLL + threadIdx.x;
    float4v v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        size_t i = base + (size_t)u * 256;
        if (i < n4) v[u] = NT ? __builtin_nontemporal_load(in + i) : in[i];
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        size_t i = base + (size_t)u * 256;
        if (i < n4) { if (NT) __builtin_nontemporal_store(v[u], out + i); else out[i] = v[u]; }
    }
}

// 4:1 read:write like quantize (read 16B, write 4B per lane)
template <int UNROLL>
__global__ __launch_bounds__(256) void quantlike_kernel(const float4v* __restrict__ in, unsigned* __restrict__ out, size_t n4) {
    size_t base = (size_t)blockIdx.x * 256 * UNROLL + threadIdx.x;
    float4v v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) { size_t i = base + (size_t)u * 256; if (i < n4) v[u] = in[i]; }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) { size_t i = base + (size_t)u * 256; if (i < n4) out[i] = __builtin_bit_cast(unsigned, v[u].x + v[u].y + v[u].z + v[u].w); }
}

// 4:1 read:write with the hint on both directions
template <int UNROLL>
__global__ __launch_bounds__(256) void quantlike_nt_kernel(const float4v* __restrict__ in, unsigned* __restrict__ out, size_t n4) {
    size_t base = (size_t)blockIdx.x * 256 * UNROLL + threadIdx.x;
    float4v v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) { size_t i = base + (size_t)u * 256; if (i < n4) v[u] = __builtin_nontemporal_load(in + i); }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        size_t i = base + (size_t)u * 256;
        if (i < n4) __builtin_nontemporal_store(__builtin_bit_cast(unsigned, v[u].x + v[u].y + v[u].z + v[u].w), out + i);
    }
}

// 2:1 read:write, the traffic of an 8-bit quantize of 16-bit elements (read 16 B, write 8 B per lane)
typedef unsigned uint2v __attribute__((ext_vector_type(2)));
template <int UNROLL, bool NT_STORE>
__global__ __launch_bounds__(256) void quantlike16_kernel(const float4v* __restrict__ in, uint2v* __restrict__ out, size_t n4) {
    size_t base = (size_t)blockIdx.x * 256 * UNROLL + threadIdx.x;
    float4v v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) { size_t i = base + (size_t)u * 256; if (i < n4) v[u] = __builtin_nontemporal_load(in + i); }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        size_t i = base + (size_t)u * 256;
        if (i >= n4) continue;
        const uint2v o = {__builtin_bit_cast(unsigned, v[u].x + v[u].y), __builtin_bit_cast(unsigned, v[u].z + v[u].w)};
        if (NT_STORE) __builtin_nontemporal_store(o, out + i); else out[i] = o;
    }
}

// The W=8 fused reduce's traffic: per lane eight dwords of codes (non-temporal), eight scales shared by 16 lanes, one
// 16-byte store (STORE: cache policy operand, 0 plain, 16 written through); every XCD walks a contiguous eighth.
typedef unsigned uint4v __attribute__((ext_vector_type(4)));
struct ReduceLike { const unsigned* codes[8]; const float* scales[8]; float* out; unsigned n4; };
template <int STORE>
__global__ __launch_bounds__(256) void reducelike_kernel(const ReduceLike a) {
    const unsigned per = gridDim.x >> 3;
    const unsigned b = blockIdx.x < (per << 3) ? (blockIdx.x & 7u) * per + (blockIdx.x >> 3) : blockIdx.x;
    const unsigned i = b * 256 + threadIdx.x;
    if (i >= a.n4) return;
    unsigned m = 0;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const __amdgpu_buffer_rsrc_t codes = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned*>(a.codes[r]), 0, a.n4 * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t scales = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(a.scales[r]), 0, a.n4 / 4, 0x00020000);
        m |= __builtin_amdgcn_raw_buffer_load_b32(codes, i * 4, 0, 2) ^ __builtin_amdgcn_raw_buffer_load_b32(scales, (i >> 4) * 4, 0, 0);
    }
    const uint4v v = {m, m + 1, m + 2, m + 3};
    __builtin_amdgcn_raw_buffer_store_b128(v, __builtin_amdgcn_make_buffer_rsrc(a.out, 0, a.n4 * 16, 0x00020000), i * 16, 0, STORE);
}

struct Timer {
    hipEvent_t a, b;
    Timer() { CK(hipEventCreate(&a)); CK(hipEventCreate(&b)); }
};

template <typename F>
double run(F launch, int iters, int nbuf) {
    Timer t;
    for (int i = 0; i < 5; ++i) launch(i % nbuf);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(t.a));
    for (int i = 0; i < iters; ++i) launch(i % nbuf);
    CK(hipEventRecord(t.b));
    CK(hipEventSynchronize(t.b));
    float ms; CK(hipEventElapsedTime(&ms, t.a, t.b));
    return ms * 1e-3 / iters;
}

// "shape" mode: the fp32 quantize's traffic on 100 MiB against (a) the workgroups that fit a CU, limited through
// an LDS allocation, with one, two or four tiles a lane in flight, and (b) a grid whose last part is cut into one-tile
// workgroups - what occupancy and the drain of coarse workgroups are worth for such a launch.
template <int UNROLL>
__global__ __launch_bounds__(256) void quantlike_lds_kernel(const float4v* __restrict__ in, unsigned* __restrict__ out, size_t n4) {
    extern __shared__ char lds[];
    size_t base = (size_t)blockIdx.x * 256 * UNROLL + threadIdx.x;
    float4v v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) { size_t i = base + (size_t)u * 256; if (i < n4) v[u] = __builtin_nontemporal_load(in + i); }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        size_t i = base + (size_t)u * 256;
        if (i < n4) __builtin_nontemporal_store(__builtin_bit_cast(unsigned, v[u].x + v[u].y + v[u].z + v[u].w), out + i);
    }
    if (n4 == 1) lds[threadIdx.x] = 1;   // keeps the allocation
}

__global__ __launch_bounds__(256) void quantlike_tail_kernel(const float4v* __restrict__ in, unsigned* __restrict__ out, size_t n4,
                                                            unsigned split) {
    if (blockIdx.x < split) {            // four tiles a lane
        size_t base = (size_t)blockIdx.x * 1024 + threadIdx.x;
        float4v v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(in + base + u * 256);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            __builtin_nontemporal_store(__builtin_bit_cast(unsigned, v[u].x + v[u].y + v[u].z + v[u].w), out + base + u * 256);
    } else {                             // one tile a lane behind them
        size_t i = (size_t)split * 1024 + (size_t)(blockIdx.x - split) * 256 + threadIdx.x;
        if (i < n4) {
            float4v v = __builtin_nontemporal_load(in + i);
            __builtin_nontemporal_store(__builtin_bit_cast(unsigned, v.x + v.y + v.z + v.w), out + i);
        }
    }
}

template <typename F>
static double best_of(F launch, int nbuf) {
    Timer t;
    for (int i = 0; i < 300; ++i) launch(i % nbuf);
    CK(hipDeviceSynchronize());
    double best = 1e9;
    for (int rep = 0; rep < 7; ++rep) {
        CK(hipEventRecord(t.a));
        for (int i = 0; i < 60; ++i) launch(i % nbuf);
        CK(hipEventRecord(t.b));
        CK(hipEventSynchronize(t.b));
        float ms; CK(hipEventElapsedTime(&ms, t.a, t.b));
        if (ms / 60 < best) best = ms / 60;
    }
    return best * 1e-3;
}

static int shape_mode() {
    const size_t bytes = (size_t)100 << 20, n4 = bytes / 16;
    const int nbuf = 6;
    std::vector<float4v*> in(nbuf); std::vector<unsigned*> out(nbuf);
    for (int i = 0; i < nbuf; ++i) { CK(hipMalloc(&in[i], bytes)); CK(hipMalloc(&out[i], bytes / 4)); CK(hipMemset(in[i], 1, bytes)); }
    const int lds_sizes[] = {0, 26 * 1024, 40 * 1024, 80 * 1024};
    CK(hipFuncSetAttribute((const void*)quantlike_lds_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024));
    CK(hipFuncSetAttribute((const void*)quantlike_lds_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024));
    CK(hipFuncSetAttribute((const void*)quantlike_lds_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024));
    for (int lds : lds_sizes)
        for (int U : {1, 2, 4}) {
            const unsigned grid = (unsigned)((n4 + 256 * U - 1) / (256 * U));
            double t = best_of([&](int k) {
                if (U == 1) hipLaunchKernelGGL(quantlike_lds_kernel<1>, dim3(grid), dim3(256), lds, 0, in[k], out[k], n4);
                if (U == 2) hipLaunchKernelGGL(quantlike_lds_kernel<2>, dim3(grid), dim3(256), lds, 0, in[k], out[k], n4);
                if (U == 4) hipLaunchKernelGGL(quantlike_lds_kernel<4>, dim3(grid), dim3(256), lds, 0, in[k], out[k], n4);
            }, nbuf);
            printf("SHAPE lds %6d B a workgroup, %d tile(s) a lane: %.2f us (%.1f %% of 8 TB/s)\n", lds, U, t * 1e6,
                   bytes * 1.25 / t / 8e12 * 100);
            fflush(stdout);
        }
    const unsigned full = (unsigned)(n4 / 1024);
    for (int pct : {100, 97, 90, 75, 50, 0}) {
        const unsigned split = (unsigned)((size_t)full * pct / 100);
        const unsigned rest = (unsigned)((n4 - (size_t)split * 1024 + 255) / 256);
        double t = best_of([&](int k) { hipLaunchKernelGGL(quantlike_tail_kernel, dim3(split + rest), dim3(256), 0, 0, in[k], out[k], n4, split); },
                           nbuf);
        printf("SHAPE four-tile workgroups for %3d %% of the data, one-tile workgroups behind: %.2f us (%.1f %% of 8 TB/s)\n", pct, t * 1e6,
               bytes * 1.25 / t / 8e12 * 100);
        fflush(stdout);
    }
    return 0;
}

// "rows" mode: the two traffic mixes the hot kernels are held to, at the caller's sizes, over > 600 MB of buffers
static int rows_mode(size_t reduce_elems, size_t quant_elems, size_t quant16_elems) {
    {
        const size_t n4 = reduce_elems / 4, groups = reduce_elems / 64;
        const size_t per_set = 8 * (reduce_elems + groups * 4) + reduce_elems * 4;
        const int sets = (int)((size_t)640000000 / per_set) + 1;
        std::vector<ReduceLike> args(sets);
        for (auto& a : args) {
            for (int r = 0; r < 8; ++r) {
                unsigned* c; float* s;
                CK(hipMalloc(&c, reduce_elems)); CK(hipMalloc(&s, groups * 4)); CK(hipMemset(c, 1, reduce_elems)); CK(hipMemset(s, 1, groups * 4));
                a.codes[r] = c; a.scales[r] = s;
            }
            CK(hipMalloc(&a.out, reduce_elems * 4)); a.n4 = (unsigned)n4;
        }
        const unsigned grid = (unsigned)((n4 + 255) / 256);
        const bool large = reduce_elems * 4 >= ((size_t)24 << 20);
        double t = run([&](int b) { if (large) reducelike_kernel<16><<<grid, 256>>>(args[b]); else reducelike_kernel<0><<<grid, 256>>>(args[b]); },
                       10 * sets, sets);
        printf("ROW reduce_like_w8 %.3f %zu\n", t * 1e6, per_set);
        for (auto& a : args) { for (int r = 0; r < 8; ++r) { CK(hipFree((void*)a.codes[r])); CK(hipFree((void*)a.scales[r])); } CK(hipFree(a.out)); }
    }
    {
        const size_t n4 = quant_elems / 4, per_set = quant_elems * 4 + quant_elems;
        const int sets = (int)((size_t)640000000 / per_set) + 1;
        std::vector<float4v*> in(sets); std::vector<unsigned*> out(sets);
        for (int i = 0; i < sets; ++i) { CK(hipMalloc(&in[i], quant_elems * 4)); CK(hipMalloc(&out[i], quant_elems)); CK(hipMemset(in[i], 1, quant_elems * 4)); }
        const unsigned grid = (unsigned)((n4 + 1023) / 1024);
        double t = run([&](int b) { quantlike_nt_kernel<4><<<grid, 256>>>(in[b], out[b], n4); }, 10 * sets, sets);
        printf("ROW quant_like_fp32 %.3f %zu\n", t * 1e6, per_set);
        for (int i = 0; i < sets; ++i) { CK(hipFree(in[i])); CK(hipFree(out[i])); }
    }
    if (quant16_elems) {   // optional third row: 16-bit elements, 8-bit codes
        const size_t n4 = quant16_elems / 8, per_set = quant16_elems * 2 + quant16_elems;
        const int sets = (int)((size_t)640000000 / per_set) + 1;
        std::vector<float4v*> in(sets); std::vector<uint2v*> out(sets);
        for (int i = 0; i < sets; ++i) { CK(hipMalloc(&in[i], quant16_elems * 2)); CK(hipMalloc(&out[i], quant16_elems)); CK(hipMemset(in[i], 1, quant16_elems * 2)); }
        const unsigned grid = (unsigned)((n4 + 1023) / 1024);
        double plain = run([&](int b) { quantlike16_kernel<4, false><<<grid, 256>>>(in[b], out[b], n4); }, 10 * sets, sets);
        double hinted = run([&](int b) { quantlike16_kernel<4, true><<<grid, 256>>>(in[b], out[b], n4); }, 10 * sets, sets);
        printf("ROW quant_like_16bit %.3f %zu\n", plain * 1e6, per_set);
        printf("ROW quant_like_16bit_nt_store %.3f %zu\n", hinted * 1e6, per_set);
    }
    return 0;
}

// "depth" mode: the plain read, write, copy and quantize-like kernels on 100 MiB buffers while the number of buffers
// (pairs) in rotation grows from 2 to 32: how much of a launch's time depends on how long ago its pages were last
// touched, for kernels that do nothing but move bytes.
static int depth_mode() {
    const size_t bytes = (size_t)100 << 20, n4 = bytes / 16;
    const int most = 32;
    std::vector<float4v*> in(most), out(most);
    for (int i = 0; i < most; ++i) { CK(hipMalloc(&in[i], bytes)); CK(hipMalloc(&out[i], bytes)); CK(hipMemset(in[i], 1, bytes)); CK(hipMemset(out[i], 0, bytes)); }
    float* flag; CK(hipMalloc(&flag, 4));
    printf("buffers in rotation (100 MiB each, a read and a write buffer per step)   read U=2   write U=4 nt   copy U=4 nt   16B in / 4B out nt   us\n");
    for (int nbuf : {2, 3, 4, 6, 8, 12, 16, 24, 32}) {
        const int iters = nbuf * 4 < 48 ? 48 : nbuf * 4;
        auto best_of3 = [&](auto launch) { double best = 1e9; for (int r = 0; r < 3; ++r) { const double t = run(launch, iters, nbuf); best = t < best ? t : best; } return best; };
        const double r = best_of3([&](int b){ read_kernel<2,false><<<(unsigned)((n4 + 511) / 512),256>>>(in[b], flag, n4); });
        const double w = best_of3([&](int b){ write_kernel<4,true><<<(unsigned)((n4 + 1023) / 1024),256>>>(out[b], n4); });
        const double c = best_of3([&](int b){ copy_kernel<4,true><<<(unsigned)((n4 + 1023) / 1024),256>>>(in[b], out[b], n4); });
        const double q = best_of3([&](int b){ quantlike_nt_kernel<4><<<(unsigned)((n4 + 1023) / 1024),256>>>(in[b], (unsigned*)out[b], n4); });
        printf("DEPTH %2d   %8.2f   %8.2f   %8.2f   %8.2f\n", nbuf, r * 1e6, w * 1e6, c * 1e6, q * 1e6); fflush(stdout);
    }
    return 0;
}

int main(int argc, char** argv) {
    if (argc > 1 && std::string(argv[1]) == "depth") return depth_mode();
    if (argc > 3 && std::string(argv[1]) == "rows") return rows_mode((size_t)atoll(argv[2]), (size_t)atoll(argv[3]), argc > 4 ? (size_t)atoll(argv[4]) : 0);
    if (argc > 1 && std::string(argv[1]) == "shape") return shape_mode();
    size_t bytes = (argc > 1 ? atol(argv[1]) : 100) * (size_t)1048576;
    int nbuf = 6;
    std::vector<float4v*> in(nbuf), out(nbuf);
    for (int i = 0; i < nbuf; ++i) { CK(hipMalloc(&in[i], bytes)); CK(hipMalloc(&out[i], bytes)); CK(hipMemset(in[i], 1, bytes)); CK(hipMemset(out[i], 0, bytes)); }
    float* flag; CK(hipMalloc(&flag, 4));
    size_t n4 = bytes / 16;
    int iters = 50;
    int cus = 256;
    printf("buffer %zu MiB x %d rotating\n", bytes >> 20, nbuf);
#define REPORT(name, nb, t) printf("%-44s %8.2f us  %8.1f GB/s (%4.1f%%)\n", name, (t)*1e6, (nb)/(t)/1e9, (nb)/(t)/8e12*100); fflush(stdout)
#define GRID(U) (unsigned)((n4 + 256 * (U) - 1) / (256 * (U)))
    { double t = run([&](int b){ read_kernel<1,false><<<GRID(1),256>>>(in[b], flag, n4); }, iters, nbuf); REPORT("read  U=1", bytes, t); }
    { double t = run([&](int b){ read_kernel<2,false><<<GRID(2),256>>>(in[b], flag, n4); }, iters, nbuf); REPORT("read  U=2", bytes, t); }
    { double t = run([&](int b){ read_kernel<4,false><<<GRID(4),256>>>(in[b], flag, n4); }, iters, nbuf); REPORT("read  U=4", bytes, t); }
    { double t = run([&](int b){ read_kernel<8,false><<<GRID(8),256>>>(in[b], flag, n4); }, iters, nbuf); REPORT("read  U=8", bytes, t); }
    { double t = run([&](int b){ read_kernel<4,true><<<GRID(4),256>>>(in[b], flag, n4); }, iters, nbuf); REPORT("read  U=4 nontemporal", bytes, t); }
    for (int mult : {2, 4, 8, 16}) {
        char name[64]; snprintf(name, 64, "read  grid-stride U=4 blocks=%d*CU", mult);
        double t = run([&](int b){ read_gs_kernel<4,false><<<cus*mult,256>>>(in[b], flag, n4); }, iters, nbuf); REPORT(name, bytes, t);
    }
    { double t = run([&](int b){ write_kernel<1,false><<<GRID(1),256>>>(out[b], n4); }, iters, nbuf); REPORT("write U=1", bytes, t); }
    { double t = run([&](int b){ write_kernel<4,false><<<GRID(4),256>>>(out[b], n4); }, iters, nbuf); REPORT("write U=4", bytes, t); }
    { double t = run([&](int b){ write_kernel<4,true><<<GRID(4),256>>>(out[b], n4); }, iters, nbuf); REPORT("write U=4 nontemporal", bytes, t); }
    { double t = run([&](int b){ copy_kernel<1,false><<<GRID(1),256>>>(in[b], out[b], n4); }, iters, nbuf); REPORT("copy  U=1", 2*bytes, t); }
    { double t = run([&](int b){ copy_kernel<4,false><<<GRID(4),256>>>(in[b], out[b], n4); }, iters, nbuf); REPORT("copy  U=4", 2*bytes, t); }
    { double t = run([&](int b){ copy_kernel<4,true><<<GRID(4),256>>>(in[b], out[b], n4); }, iters, nbuf); REPORT("copy  U=4 nontemporal", 2*bytes, t); }
    { double t = run([&](int b){ copy_kernel<8,true><<<GRID(8),256>>>(in[b], out[b], n4); }, iters, nbuf); REPORT("copy  U=8 nontemporal", 2*bytes, t); }
    { double t = run([&](int b){ quantlike_kernel<4><<<GRID(4),256>>>(in[b], (unsigned*)out[b], n4); }, iters, nbuf); REPORT("quant-like 16B in / 4B out U=4", bytes + bytes/4, t); }
    { double t = run([&](int b){ quantlike_kernel<8><<<GRID(8),256>>>(in[b], (unsigned*)out[b], n4); }, iters, nbuf); REPORT("quant-like 16B in / 4B out U=8", bytes + bytes/4, t); }
    { double t = run([&](int b){ quantlike_nt_kernel<4><<<GRID(4),256>>>(in[b], (unsigned*)out[b], n4); }, iters, nbuf); REPORT("quant-like 16B in / 4B out U=4 nontemporal", bytes + bytes/4, t); }
    { double t = run([&](int b){ CK(hipMemcpyAsync(out[b], in[b], bytes, hipMemcpyDeviceToDevice, 0)); }, iters, nbuf); REPORT("hipMemcpyAsync D2D", 2*bytes, t); }
    return 0;
}
