// The 4-bit code books of the reference's CUDA extension (ccdl_comm/csrc/quantization/inner.cuh:9-35) and, built
// from them at compile time, a one-lookup form of its encoder.
//
// The reference encodes t = v / scale by a search for the largest entry not above t followed by a rounding step,
// `entry + (t - book[entry] > (book[entry + 1] - book[entry]) * 0.5f)` (inner.cuh:74-118).  For one book that is a
// non-decreasing step function of t with fourteen steps.  The places of the steps (the smallest float at which the
// code becomes k + 1) are found here by bisection over the float line with the reference's own arithmetic, and
// [-1, 1] is cut into 256 cells of width 1/128, none of which holds two steps.  A cell stores the code at its left
// end and the step inside it, if any, so that on the device
//     code(t) = cell.base + (t >= cell.threshold),   cell = cells[(unsigned)fma(t, 128, 128)]
// for every finite t in [-1, 1].  tests/native/check_book_cells.cpp compares the two forms on every such float.
// Plain C++17 (host and device): no HIP types.
#pragma once
#include <cstdint>

namespace lbc {
namespace book_cells {

constexpr int kBooks = 4;
constexpr int kCells = 257;   // (unsigned)(t * 128 + 128) for t in [-1, 1] is 0..256

// entry 15 is never produced by the encoder
struct Books {
    float value[kBooks][16];
};
constexpr Books kBookSet = {{
    {-1.0f, -0.815410147f, -0.655160150f, -0.510228027f, -0.375324982f, -0.246951370f, -0.122538030f, 0.0f,
     0.122538030f, 0.246951370f, 0.375324982f, 0.510228027f, 0.655160150f, 0.815410147f, 1.0f, __builtin_inff()},
    {-1.0f, -0.85714286f, -0.71428571f, -0.57142857f, -0.42857143f, -0.28571429f, -0.14285714f, 0.0f,
     0.14285714f, 0.28571429f, 0.42857143f, 0.57142857f, 0.71428571f, 0.85714286f, 1.0f, __builtin_inff()},
    {-1.0f, -0.5f, -0.25f, -0.125f, -0.0625f, -0.03125f, -0.015625f, 0.0f,
     0.015625f, 0.03125f, 0.0625f, 0.125f, 0.25f, 0.5f, 1.0f, __builtin_inff()},
    {-1.0f, -0.6666666666666666f, -0.5f, -0.3333333333333333f, -0.25f, -0.16666666666666666f, -0.125f, 0.0f,
     0.125f, 0.16666666666666666f, 0.25f, 0.3333333333333333f, 0.5f, 0.6666666666666666f, 1.0f, __builtin_inff()},
}};

struct Cell {
    float threshold;   // the code rises by one at this value; +inf when the cell holds no step
    uint32_t base;     // the code at the cell's left end
};
struct Table {
    Cell cell[kCells];
};
struct Tables {
    Table book[kBooks];
};

// The reference's encoder for a number t (not NaN): search, then rounding.
constexpr int searched_code(const float (&book)[16], float t) {
    int at = 0;
    for (int entry = 1; entry <= 14; ++entry)
        if (!(t < book[entry])) at = entry;
    if (at == 14) return 14;   // the gap to entry 15 is infinite: never rounds up
    const float low = book[at], gap = book[at + 1] - low, excess = t - low;
    return at + (excess > gap * 0.5f ? 1 : 0);
}

// Floats as unsigned keys in the order of their values, and back.
constexpr uint32_t key_of(float f) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, f);
    return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}
constexpr float float_of(uint32_t key) {
    return __builtin_bit_cast(float, (key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
}

// t * 128 is exact, so this is the device's single-rounding fma(t, 128, 128).
constexpr int cell_of(float t) { return static_cast<int>(t * 128.0f + 128.0f); }

// The smallest float in [-1, 1] whose code is above k.
constexpr float step_after(const float (&book)[16], int k) {
    uint32_t below = key_of(-1.0f), reached = key_of(1.0f);   // code(-1) = 0 <= k < 14 = code(1)
    while (reached - below > 1) {
        const uint32_t middle = below + (reached - below) / 2;
        if (searched_code(book, float_of(middle)) > k) reached = middle;
        else below = middle;
    }
    return float_of(reached);
}

constexpr Table make_table(const float (&book)[16]) {
    Table table{};
    float step[14]{};
    for (int k = 0; k < 14; ++k) step[k] = step_after(book, k);
    for (int i = 0; i < kCells; ++i) {
        uint32_t base = 0;
        float threshold = __builtin_inff();
        for (int k = 0; k < 14; ++k) {
            if (cell_of(step[k]) < i) ++base;
            else if (cell_of(step[k]) == i) threshold = step[k];
        }
        table.cell[i] = Cell{threshold, base};
    }
    return table;
}

// One step per cell at most, or the lookup would miss a step.
constexpr bool steps_in_separate_cells(const float (&book)[16]) {
    int previous = -1;
    for (int k = 0; k < 14; ++k) {
        const int cell = cell_of(step_after(book, k));
        if (cell <= previous) return false;
        previous = cell;
    }
    return true;
}

constexpr Tables kTables = {{make_table(kBookSet.value[0]), make_table(kBookSet.value[1]), make_table(kBookSet.value[2]),
                               make_table(kBookSet.value[3])}};
static_assert(steps_in_separate_cells(kBookSet.value[0]) && steps_in_separate_cells(kBookSet.value[1]) &&
                  steps_in_separate_cells(kBookSet.value[2]) && steps_in_separate_cells(kBookSet.value[3]),
              "a cell of width 1/128 holds two steps of a code book");

// The lookup, as the device does it.
constexpr int cell_code(const Table &table, float t) {
    const Cell &cell = table.cell[cell_of(t)];
    return static_cast<int>(cell.base) + (t >= cell.threshold ? 1 : 0);
}

}  // namespace book_cells
}  // namespace lbc
