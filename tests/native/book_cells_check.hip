// Device check of the one-lookup code-book encoder (lowbit_comm_amd/csrc/code_book_cells.h): for each of the four
// books and every float t in [-1, 1], the lookup as the quantize kernel does it - the cell of fma(t, 128, 128)
// converted to an unsigned integer, then `base + (t >= threshold)` - against the search and rounding step it stands
// for (ccdl_comm/csrc/quantization/inner.cuh:74-118), both evaluated on the device.  Prints "MISMATCHES n";
// exit status 1 when n is not 0.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../lowbit_comm_amd/csrc/code_book_cells.h"

namespace bc = lbc::book_cells;

__constant__ bc::Books kBooks = bc::kBookSet;
__constant__ bc::Tables kCells = bc::kTables;

__global__ void compare(int book_index, uint32_t first_key, uint64_t count, unsigned long long *bad) {
    const float *book = kBooks.value[book_index];
    const bc::Cell *cells = kCells.book[book_index].cell;
    unsigned long long mine = 0;
    for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < count; i += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t key = first_key + (uint32_t)i;
        const float t = __uint_as_float((key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
        int at = 0;
        for (int step = 8; step >= 1; step >>= 1) {
            const int mid = at + step;
            if (mid < 15 && !(t < book[mid])) at = mid;
        }
        const float low = book[at], gap = book[at + 1] - low, excess = t - low;
        const int searched = at + (excess > gap * 0.5f ? 1 : 0);
        const bc::Cell cell = cells[static_cast<uint32_t>(__builtin_fmaf(t, 128.0f, 128.0f))];
        const int looked_up = static_cast<int>(cell.base) + (t >= cell.threshold ? 1 : 0);
        mine += searched != looked_up;
    }
    if (mine) atomicAdd(bad, mine);
}

int main() {
    unsigned long long *bad, total = 0, floats = 0;
    if (hipMalloc(&bad, sizeof(*bad)) != hipSuccess) return 2;
    const uint32_t first = bc::key_of(-1.0f), last = bc::key_of(1.0f);
    const uint64_t count = (uint64_t)last - first + 1;
    for (int b = 0; b < bc::kBooks; ++b) {
        unsigned long long h = 0;
        if (hipMemcpy(bad, &h, sizeof(h), hipMemcpyHostToDevice) != hipSuccess) return 2;
        hipLaunchKernelGGL(compare, dim3(8192), dim3(256), 0, 0, b, first, count, bad);
        if (hipDeviceSynchronize() != hipSuccess) return 2;
        if (hipMemcpy(&h, bad, sizeof(h), hipMemcpyDeviceToHost) != hipSuccess) return 2;
        printf("book %d: %llu floats, %llu mismatches\n", b, (unsigned long long)count, h);
        total += h;
        floats += count;
    }
    printf("CHECKED %llu\nMISMATCHES %llu\n", floats, total);
    return total ? 1 : 0;
}
