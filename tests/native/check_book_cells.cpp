// Host check of the one-lookup code-book encoder (lowbit_comm_amd/csrc/code_book_cells.h): on every float in
// [-1, 1], for each of the four books, the cell lookup must give the code of the search-and-round form
// (ccdl_comm/csrc/quantization/inner.cuh:74-118), evaluated here at run time with ordinary float arithmetic.
// Build: g++ -O2 -std=c++17 -ffp-contract=off -fopenmp check_book_cells.cpp.  Prints "MISMATCHES n".
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../lowbit_comm_amd/csrc/code_book_cells.h"

namespace bc = lbc::book_cells;

static int searched(const float *book, float t) {
    int at = 0;
    for (int step = 8; step >= 1; step >>= 1) {       // the halving search of the kernels
        const int mid = at + step;
        if (mid < 15 && !(t < book[mid])) at = mid;
    }
    const volatile float low = book[at];
    const volatile float gap = book[at + 1] - low;
    const volatile float excess = t - low;
    return at + (excess > gap * 0.5f ? 1 : 0);
}

int main(int argc, char **argv) {
    const uint32_t stride = argc > 1 ? static_cast<uint32_t>(std::strtoul(argv[1], nullptr, 10)) : 1u;
    const uint32_t first = bc::key_of(-1.0f), last = bc::key_of(1.0f);
    unsigned long long mismatches = 0, checked = 0;
    for (int b = 0; b < bc::kBooks; ++b) {
        const float *book = bc::kBookSet.value[b];
        const bc::Table &table = bc::kTables.book[b];
        unsigned long long bad = 0, seen = 0;
#pragma omp parallel for reduction(+ : bad, seen) schedule(static)
        for (long long k = first; k <= static_cast<long long>(last); k += stride) {
            const float t = bc::float_of(static_cast<uint32_t>(k));
            const float u = __builtin_fmaf(t, 128.0f, 128.0f);
            const bc::Cell &cell = table.cell[static_cast<uint32_t>(u)];
            const int got = static_cast<int>(cell.base) + (t >= cell.threshold ? 1 : 0);
            bad += got != searched(book, t);
            ++seen;
        }
        // every step itself and the float before it, whatever the stride
        for (int i = 0; i < bc::kCells; ++i) {
            const float at = table.cell[i].threshold;
            if (at > 1.0f) continue;
            const float before = bc::float_of(bc::key_of(at) - 1);
            bad += bc::cell_code(table, at) != searched(book, at);
            bad += bc::cell_code(table, before) != searched(book, before);
            bad += bc::cell_code(table, at) != bc::cell_code(table, before) + 1;
            seen += 3;
        }
        std::printf("book %d: %llu floats, %llu mismatches\n", b, seen, bad);
        mismatches += bad;
        checked += seen;
    }
    std::printf("CHECKED %llu\nMISMATCHES %llu\n", checked, mismatches);
    return mismatches ? 1 : 0;
}
