// Distributed vector sum, the workload of the reference's examples/thread-group.cu:31-47: every PE adds
// its slices of x and y, then the partial sums of all PEs are concatenated on every PE with fcollect -
// once called by the whole block (nvshmemx_int_fcollect_block: all threads share the copy), once by
// thread 0 alone (nvshmem_int_fcollect).  With x[i] = 1000 p + i and y[i] = i on PE p every PE must end
// with sum[p n + i] = 1000 p + 2 i.
#include "example_util.hpp"

__global__ void distributed_vector_sum(const int *x, const int *y, int *partial_sum, int *sum, int use_threadgroup) {
    const int me = nvshmem_my_pe();
    const int index = threadIdx.x, nelems = blockDim.x;
    ((int *)nvshmem_ptr(partial_sum, me))[index] =
        ((const int *)nvshmem_ptr(x, me))[index] + ((const int *)nvshmem_ptr(y, me))[index];
    if (use_threadgroup) {
        nvshmemx_int_fcollect_block(NVSHMEM_TEAM_WORLD, sum, partial_sum, nelems);
    } else {
        __syncthreads();  // thread 0 sends what the other threads wrote
        if (index == 0) nvshmem_int_fcollect(NVSHMEM_TEAM_WORLD, sum, partial_sum, nelems);
    }
}

int main() {
    nvshmem_init();
    const int np = nvshmem_n_pes();
    const int nthreads = 512;
    int *x = (int *)nvshmem_malloc(sizeof(int) * nthreads);
    int *y = (int *)nvshmem_malloc(sizeof(int) * nthreads);
    int *partial_sum = (int *)nvshmem_malloc(sizeof(int) * nthreads);
    int *sum = (int *)nvshmem_malloc(sizeof(int) * nthreads * np);
    for (int pe = 0; pe < np; ++pe) {
        std::vector<int> hx(nthreads), hy(nthreads);
        for (int i = 0; i < nthreads; ++i) {
            hx[i] = 1000 * pe + i;
            hy[i] = i;
        }
        store(x, hx, pe);
        store(y, hy, pe);
    }
    long errors = 0;
    for (int use_threadgroup = 1; use_threadgroup >= 0; --use_threadgroup) {
        for (int pe = 0; pe < np; ++pe) store(sum, std::vector<int>((size_t)nthreads * np, -1), pe);
        void *args[] = {&x, &y, &partial_sum, &sum, &use_threadgroup};
        NVSHMEM_CHECK(nvshmemx_collective_launch((const void *)distributed_vector_sum, dim3(1), dim3(nthreads), args,
                                                 0, nullptr));
        HIP_CHECK(hipDeviceSynchronize());
        for (int pe = 0; pe < np; ++pe) {
            const std::vector<int> got = fetch(sum, (size_t)nthreads * np, pe);
            for (int p = 0; p < np; ++p)
                for (int i = 0; i < nthreads; ++i) errors += got[(size_t)p * nthreads + i] != 1000 * p + 2 * i;
        }
    }
    nvshmem_free(x);
    nvshmem_free(y);
    nvshmem_free(partial_sum);
    nvshmem_free(sum);
    return finish("thread_group", errors);
}
