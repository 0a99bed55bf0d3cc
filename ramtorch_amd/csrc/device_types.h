// Records the update kernels read from device memory, and the launch geometry
// shared by host and device code.  gfx950 only.
#pragma once
#include <stdint.h>

#include "../../include/ramtorch_sr_adamw.h"

namespace rt {

constexpr int kThreads = 256;                       // 4 wavefronts of 64
constexpr int kVec = 8;                             // elements per lane per vector (128 bit of bf16)
constexpr int kItersPerChunk = 4;                   // vectors per lane per chunk
constexpr uint32_t kChunkElems = kThreads * kVec * kItersPerChunk;  // 8192

// DevTensor.flags
constexpr uint32_t kFlagAligned = 1u;  // every array pointer of the tensor is 16-byte aligned
constexpr uint32_t kFlagRowwise = 2u;  // centralization with the row means taken inside the update kernel (row_mean == 0)

// One tensor (or contiguous piece) as the kernels see it; 128 bytes so that a
// record never straddles more cache lines than it has to.
struct alignas(16) DevTensor {
    uint64_t p, g, m, v;        // device addresses
    uint64_t np, nm, nv;        // explicit noise (uint16 per element) or 0
    uint64_t dp, dm, dv;        // optional fp32 debug outputs or 0
    uint64_t row_mean;          // fp32 row means for centralization or 0
    uint64_t numel;
    uint64_t block_base;        // elem_offset / 8: first Philox block of this piece
    uint64_t row_len;
    uint32_t tensor_id4;        // tensor_id * 4; + {0,1,2} selects p / m / v noise
    uint32_t set_idx;           // index into the DevScalars array
    uint32_t flags;
    uint32_t dtypes;            // p | g << 2 | m << 4 | v << 6 (RT_DT_*), read by the runtime-typed kernel
};
static_assert(sizeof(DevTensor) == 128, "DevTensor layout");

// rt_scalars of one param group at one step count, plus that step (Philox counter word 3).
struct alignas(16) DevScalars {
    rt_scalars s;
    uint32_t step;
    uint32_t pad[3];
};
static_assert(sizeof(DevScalars) == 64, "DevScalars layout");

// One workgroup's unit of work in the generic, runtime-typed and norm kernels: chunk `chunk`
// (kChunkElems elements) of tensor `tensor`.
struct ChunkRef {
    uint32_t tensor;
    uint32_t chunk;
};

// Fast kernel: a workgroup owns one unit of kFastUnitElems consecutive elements of one tensor.
// Which tensor is found by searching a list with one entry per tensor that has whole units: the
// index of its first unit within the launch (ascending), next to a copy of its DevTensor record at
// the same position.  A few hundred bytes for a transformer's parameter set, so the search runs
// out of cache, where a per-workgroup table entry would be a fresh HBM line.
// (Units of two or four chunks per workgroup were measured 1.5 % and 2.5 % slower on the 8B set.)
constexpr int kFastIters = kItersPerChunk;           // vectors per lane per fast unit
constexpr uint32_t kFastUnitElems = kThreads * kVec * kFastIters;

// Piece kernel: a wavefront owns one piece of at most kPieceElems consecutive elements -- a whole
// short tensor, or part of what a long tensor leaves over after its whole fast units.  The record
// is self-contained (no DevTensor lookup), so a wave's first vector load waits for one table read.
constexpr uint32_t kPieceElems = 64 * kVec;  // 512: one 128-bit vector per lane
struct alignas(16) PieceRef {
    uint64_t p, g, m, v;   // device addresses of the piece's first element
    uint64_t block;        // Philox block of the piece's first element ((elem_offset + start) / 8)
    uint32_t count;        // 1 .. kPieceElems
    uint32_t tensor_id4;
    uint32_t set_idx;
    uint32_t pad[3];
};
static_assert(sizeof(PieceRef) == 64, "PieceRef layout");

// Kernel arguments of the update kernels (passed by value).
struct LaunchArgs {
    const DevTensor* tensors;
    const DevScalars* sets;
    const uint32_t* first;          // fast kernel: first unit of each of its tensors, ascending
    const DevTensor* fast_tensors;  // fast kernel: the tensors' records, same order as `first`
    const PieceRef* pieces;  // piece part of the fast kernel
    const ChunkRef* chunks;  // generic / runtime-typed kernels
    const float* clip_coef;  // optional device float: grads are multiplied by it
    const uint32_t* skip;    // optional device flag: non-zero leaves everything untouched
    uint32_t n_ranges, n_pieces, n_piece_wgs;
    uint32_t piece_rate;     // see sr_adamw_fast_kernel: how piece workgroups are spread over the grid
    uint32_t seed_lo, seed_hi;
    uint32_t use_ks;         // every tensor of the launch uses one DevScalars: `ks`, no table read
    uint32_t n_rows;         // row-wise kernel: rows in the launch
    DevScalars ks;
};

}  // namespace rt
