// Test helper (not part of the product): raw 32-bit draws of rocRAND's Philox4x32-10 device generator, which AMD
// documents as producing cuRAND's sequence for the same (seed, subsequence, offset).  The GPU test holds the
// codec's own counter-mode Philox stream against it.
#include <hip/hip_runtime.h>
#include <rocrand/rocrand_kernel.h>

#include <cstdint>

__global__ void draws_kernel(unsigned long long seed, const unsigned long long *subsequences, int rows,
                             unsigned long long offset, int count, uint32_t *out) {
    const int row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows) return;
    rocrand_state_philox4x32_10 state;
    rocrand_init(seed, subsequences[row], offset, &state);
    for (int j = 0; j < count; ++j) out[static_cast<int64_t>(row) * count + j] = rocrand(&state);
}

extern "C" int rocrand_philox_draws(unsigned long long seed, const unsigned long long *subsequences, int rows,
                                    unsigned long long offset, int count, uint32_t *out, void *stream) {
    if (rows <= 0 || count <= 0) return 0;
    hipLaunchKernelGGL(draws_kernel, dim3((rows + 63) / 64), dim3(64), 0, static_cast<hipStream_t>(stream), seed,
                       subsequences, rows, offset, count, out);
    return static_cast<int>(hipGetLastError());
}
