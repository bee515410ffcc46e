// Layout of a grid that carries several independent stages of a bucket stream (a quantize, a reduce, a decode):
// every stage owns a run of consecutive block indices, cut into `rows` rows of `stride` slots of which the first
// `grid_x` are live (a row is one destination chunk of the quantize, or one shard of the decode; the reduce has one
// row).  A stage's body sees (block_x, grid_x, row) exactly as its stand-alone kernel sees (blockIdx.x, gridDim.x,
// blockIdx.y).
//
// Workgroups are dealt to the chip's eight XCDs by the low three bits of their index, and the stage bodies give each
// XCD one contiguous eighth of a row on that assumption (xcd_contiguous_block).  So every run starts at a multiple of
// 8 and every row has a multiple of 8 slots: block_x and the hardware index then agree in those bits for every row of
// every stage.  The surplus slots (fewer than 8 per row) return at once.
#pragma once

#include <stdint.h>

namespace lbc {

struct StepSegment {
    unsigned begin;    // first block index of the stage, a multiple of 8
    unsigned stride;   // slots per row, a multiple of 8, >= grid_x
    unsigned grid_x;   // live blocks per row
    unsigned rows;     // 0: the stage is absent
};

inline int64_t step_round_up8(int64_t v) { return (v + 7) & ~int64_t{7}; }

// Slots a stage of `rows` rows of `grid_x` blocks takes.
inline int64_t step_segment_slots(int64_t grid_x, int64_t rows) { return step_round_up8(grid_x) * rows; }

// Appends a stage at block index `cursor` (a multiple of 8) and moves the cursor past it.
inline StepSegment step_segment_at(int64_t &cursor, int64_t grid_x, int64_t rows) {
    StepSegment s{static_cast<unsigned>(cursor), static_cast<unsigned>(step_round_up8(grid_x)),
                  static_cast<unsigned>(grid_x), static_cast<unsigned>(grid_x > 0 ? rows : 0)};
    cursor += static_cast<int64_t>(s.stride) * s.rows;
    return s;
}

#if defined(__HIPCC__)
// True when block `b` belongs to the stage; block_x may be a surplus slot (>= grid_x), which the caller lets return.
__device__ __forceinline__ bool step_segment_holds(const StepSegment &s, unsigned b, unsigned &block_x, unsigned &row) {
    const unsigned local = b - s.begin;                  // wraps to a huge value for blocks before the stage
    if (local >= s.stride * s.rows) return false;
    // The quotient is the same in every lane, but the division runs on the vector unit and leaves it in a vector
    // register; from there every address the stage derives from (block_x, row) would be vector arithmetic in vector
    // registers (the quantize of a 16-bit bucket then holds 104 of them instead of 78, that of an fp32 bucket 72
    // instead of 48).  Handed back to a scalar register, the stage body compiles as in its stand-alone kernel.
    row = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(local / s.stride)));
    block_x = local - row * s.stride;
    return true;
}
#endif

}  // namespace lbc
