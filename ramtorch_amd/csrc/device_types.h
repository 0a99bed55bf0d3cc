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

// One workgroup's unit of work: chunk `chunk` (kChunkElems elements) of tensor `tensor`.
struct ChunkRef {
    uint32_t tensor;
    uint32_t chunk;
};

}  // namespace rt
