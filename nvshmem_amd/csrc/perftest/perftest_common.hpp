// Host-side argument checks shared by the perftest drivers.  A kernel that is handed a range
// outside the symmetric heap would fault the GPU, so every driver validates first.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdio>

#include "nvshmem.h"

namespace perftest {

// Also makes sure this library's device state blocks are populated: it may have been loaded after
// nvshmem_init, and its kernels are started with plain launches.
inline bool ready() {
    if (nvshmemx_init_status() == NVSHMEM_STATUS_IS_INITIALIZED)
        return nvshmemx_amd_module_init() == NVSHMEMX_SUCCESS;
    fprintf(stderr, "nvshmem_perftest: nvshmem is not initialised\n");
    return false;
}

inline bool check_launch(int blocks, int threads) {
    if (blocks >= 1 && blocks <= (1 << 22) && threads >= 1 && threads <= 1024) return true;
    fprintf(stderr, "nvshmem_perftest: bad launch shape: %d blocks x %d threads\n", blocks, threads);
    return false;
}

// [p, p+bytes) must be symmetric memory inside one PE slice.
inline bool check_range(const void *p, size_t bytes) {
    const char *first = (const char *)nvshmem_ptr(p, 0);
    if (!first) {
        fprintf(stderr, "nvshmem_perftest: %p is not a symmetric address\n", p);
        return false;
    }
    if (bytes == 0) return true;
    const char *last = (const char *)nvshmem_ptr((const char *)p + (bytes - 1), 0);
    if (!last || (size_t)(last - first) != bytes - 1) {
        fprintf(stderr, "nvshmem_perftest: range [%p, +%zu) leaves the PE's heap slice\n", p, bytes);
        return false;
    }
    return true;
}

inline int launch_status(const char *what) {
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) return 0;
    fprintf(stderr, "nvshmem_perftest: %s launch failed: %s\n", what, hipGetErrorString(e));
    return NVSHMEMX_ERROR_INTERNAL;
}

}  // namespace perftest
