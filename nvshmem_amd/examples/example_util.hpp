// Shared by the example programs: error checks and access to every PE's copy of a symmetric object.
// The host thread stands for all PEs here, so the "if (recv[i] != expected)" loop that a reference
// example runs once per process runs once per PE in the same process.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "nvshmem.h"
#include "nvshmemx.h"

#define HIP_CHECK(stmt)                                                                           \
    do {                                                                                          \
        hipError_t err_ = (stmt);                                                                 \
        if (err_ != hipSuccess) {                                                                 \
            fprintf(stderr, "%s:%d: %s failed: %s\n", __FILE__, __LINE__, #stmt, hipGetErrorString(err_)); \
            exit(1);                                                                              \
        }                                                                                         \
    } while (0)

#define NVSHMEM_CHECK(stmt)                                                                       \
    do {                                                                                          \
        int rc_ = (stmt);                                                                         \
        if (rc_ != 0) {                                                                           \
            fprintf(stderr, "%s:%d: %s returned %d: %s\n", __FILE__, __LINE__, #stmt, rc_,        \
                    nvshmemx_amd_last_error());                                                   \
            exit(1);                                                                              \
        }                                                                                         \
    } while (0)

template <typename T>
std::vector<T> fetch(const T *sym, size_t n, int pe) {
    std::vector<T> host(n);
    HIP_CHECK(hipMemcpy(host.data(), nvshmem_ptr(sym, pe), n * sizeof(T), hipMemcpyDeviceToHost));
    return host;
}

template <typename T>
void store(T *sym, const std::vector<T> &host, int pe) {
    HIP_CHECK(hipMemcpy(nvshmem_ptr(sym, pe), host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
}

inline int finish(const char *name, long errors) {
    nvshmem_finalize();
    printf("%s: %s\n", name, errors ? "FAILED" : "PASSED");
    return errors ? 1 : 0;
}
