/*
 * nvshmemx.h - extension part of the API (scoped _warp/_block calls, _on_stream calls, signals,
 * collective launch).  Stands where the reference's src/include/nvshmemx.h:15-31 stands.
 */
#ifndef NVSHMEMX_H
#define NVSHMEMX_H

#include "nvshmem.h"

#if defined(__HIPCC__)
/* The reference's C++ signature (src/device/launch/collective_launch.cpp:209-212) over the C ABI. */
static inline __host__ int nvshmemx_collective_launch(const void *func, dim3 grid, dim3 block,
                                                      void **args, size_t shared_mem,
                                                      hipStream_t stream) {
    return nvshmemx_amd_collective_launch(func, grid.x, grid.y, grid.z, block.x, block.y, block.z,
                                          args, shared_mem, (nvshmemx_stream_t)stream);
}
static inline __host__ int nvshmemx_collective_launch_query_gridsize(const void *func, dim3 block,
                                                                     void **args, size_t shared_mem,
                                                                     int *gridsize) {
    (void)args;
    return nvshmemx_amd_collective_launch_query_gridsize(func, block.x, block.y, block.z,
                                                         shared_mem, gridsize);
}
#endif

#endif
