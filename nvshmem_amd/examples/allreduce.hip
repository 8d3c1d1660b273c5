// Sum allreduce three ways with the known answer of the reference's examples/ring-reduce.cu:209,242-248
// and examples/user-buffer.cu:141-152 - every PE contributes src[i] = i, every PE must end with
// dst[i] = i * npes: (1) inside a kernel with nvshmemx_int_sum_reduce_block, (2) from the host on a
// stream with nvshmemx_float_sum_reduce_on_stream, (3) on a team made of the even PEs.
#include "example_util.hpp"

__global__ void reduce_in_kernel(int *dst, const int *src, size_t n) {
    nvshmemx_int_sum_reduce_block(NVSHMEM_TEAM_WORLD, dst, src, n);
}

int main() {
    nvshmem_init();
    const int np = nvshmem_n_pes();
    const size_t n = 100000;
    int *isrc = (int *)nvshmem_malloc(n * sizeof(int)), *idst = (int *)nvshmem_malloc(n * sizeof(int));
    float *fsrc = (float *)nvshmem_malloc(n * sizeof(float)), *fdst = (float *)nvshmem_malloc(n * sizeof(float));
    std::vector<int> iota_i(n);
    std::vector<float> iota_f(n);
    for (size_t i = 0; i < n; ++i) iota_i[i] = (int)i, iota_f[i] = (float)(i % 1000);
    for (int pe = 0; pe < np; ++pe) store(isrc, iota_i, pe), store(fsrc, iota_f, pe);
    long errors = 0;

    void *args[] = {&idst, &isrc, (void *)&n};
    NVSHMEM_CHECK(nvshmemx_collective_launch((const void *)reduce_in_kernel, dim3(1), dim3(512), args, 0, nullptr));
    nvshmem_barrier_all();
    for (int pe = 0; pe < np; ++pe) {
        const std::vector<int> got = fetch(idst, n, pe);
        for (size_t i = 0; i < n; ++i) errors += got[i] != (int)i * np;
    }

    hipStream_t stream;
    HIP_CHECK(hipStreamCreate(&stream));
    NVSHMEM_CHECK(nvshmemx_float_sum_reduce_on_stream(NVSHMEM_TEAM_WORLD, fdst, fsrc, n, stream));
    HIP_CHECK(hipStreamSynchronize(stream));
    for (int pe = 0; pe < np; ++pe) {
        const std::vector<float> got = fetch(fdst, n, pe);
        for (size_t i = 0; i < n; ++i) errors += got[i] != (float)(i % 1000) * np;  // small integers: exact
    }

    nvshmem_team_t even = NVSHMEM_TEAM_INVALID;
    NVSHMEM_CHECK(nvshmem_team_split_strided(NVSHMEM_TEAM_WORLD, 0, 2, (np + 1) / 2, nullptr, 0, &even));
    HIP_CHECK(hipMemsetAsync(nvshmem_ptr(fdst, 0), 0, n * sizeof(float), stream));
    NVSHMEM_CHECK(nvshmemx_float_sum_reduce_on_stream(even, fdst, fsrc, n, stream));
    HIP_CHECK(hipStreamSynchronize(stream));
    {
        const std::vector<float> got = fetch(fdst, n, 0);
        for (size_t i = 0; i < n; ++i) errors += got[i] != (float)(i % 1000) * ((np + 1) / 2);
    }
    nvshmem_team_destroy(even);
    HIP_CHECK(hipStreamDestroy(stream));
    nvshmem_free(isrc), nvshmem_free(idst), nvshmem_free(fsrc), nvshmem_free(fdst);
    return finish("allreduce", errors);
}
