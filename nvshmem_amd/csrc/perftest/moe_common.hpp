// Helpers shared by the translation units of the MoE token shuffle kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "nvshmemx.h"

namespace {

// A routing entry that points outside the receive buffer is skipped instead of written.
__device__ __forceinline__ bool row_ok(int pe, int64_t row, int np, size_t cap_rows) {
    return (unsigned)pe < (unsigned)np && (uint64_t)row < (uint64_t)cap_rows;
}

// The wavefront's index in its block as a scalar (the same for every lane of a wavefront): it keeps row
// indices, routing entries and the addresses derived from them in scalar registers.
__device__ __forceinline__ unsigned wave_in_block() {
    return __builtin_amdgcn_readfirstlane(threadIdx.x / NVSHMEMI_WARP_SIZE);
}
// The same value left in a vector register: the routing entries are then fetched with vector loads.  The
// kernel that pushes its rows with plain puts and signals once per block is 5 % faster that way (its few
// long-lived wavefronts stream the tables through the small scalar cache otherwise), the others are not.
__device__ __forceinline__ unsigned wave_in_block_per_lane() { return threadIdx.x / NVSHMEMI_WARP_SIZE; }

}  // namespace

namespace perftest {
// moe_rowsignal.hip: collective launch of the dispatch kernel that signals every row; `args` are the
// kernel's twelve arguments in order.
int launch_moe_rowsignal(bool warp, int blocks_per_pe, int threads, void **args, hipStream_t stream);
}  // namespace perftest
