// Local kernels and a collective chained on one stream, the shape of the reference's
// examples/on-stream.cu: every PE sums its own input, the partial sums are combined with
// nvshmemx_int_sum_reduce_on_stream, and a second kernel on every PE acts on the total - all
// ordered by the stream, no host synchronisation in between.
#include "example_util.hpp"

constexpr int kInputs = 512, kThreshold = 42, kCorrection = 7;

// launched with grid (1, 1, npes): block z works on PE z's copies, which nvshmem_my_pe() reports
__global__ void accumulate(int *input, int *partial) {
    const int me = nvshmem_my_pe();
    int *in = (int *)nvshmem_ptr(input, me), *sum = (int *)nvshmem_ptr(partial, me);
    if (threadIdx.x == 0) *sum = 0;
    __syncthreads();
    atomicAdd(sum, in[threadIdx.x]);
}

__global__ void correct_and_accumulate(int *input, int *partial, const int *total) {
    const int me = nvshmem_my_pe();
    int *in = (int *)nvshmem_ptr(input, me), *sum = (int *)nvshmem_ptr(partial, me);
    if (*(const int *)nvshmem_ptr(total, me) > kThreshold) in[threadIdx.x] -= kCorrection;
    if (threadIdx.x == 0) *sum = 0;
    __syncthreads();
    atomicAdd(sum, in[threadIdx.x]);
}

int main() {
    nvshmem_init();
    const int np = nvshmem_n_pes();
    int *input = (int *)nvshmem_malloc(kInputs * sizeof(int));
    int *partial = (int *)nvshmem_malloc(sizeof(int)), *total = (int *)nvshmem_malloc(sizeof(int));
    for (int pe = 0; pe < np; ++pe) store(input, std::vector<int>(kInputs, pe + 1), pe);
    hipStream_t stream;
    HIP_CHECK(hipStreamCreate(&stream));
    const dim3 every_pe(1, 1, np);
    hipLaunchKernelGGL(accumulate, every_pe, dim3(kInputs), 0, stream, input, partial);
    NVSHMEM_CHECK(nvshmemx_int_sum_reduce_on_stream(NVSHMEM_TEAM_WORLD, total, partial, 1, stream));
    hipLaunchKernelGGL(correct_and_accumulate, every_pe, dim3(kInputs), 0, stream, input, partial, total);
    HIP_CHECK(hipStreamSynchronize(stream));
    // PE p: 512 inputs of p + 1; the total is 512 * np (np + 1) / 2 > 42, so every input loses 7
    const int want_total = kInputs * np * (np + 1) / 2;
    long errors = 0;
    for (int pe = 0; pe < np; ++pe) {
        errors += fetch(total, 1, pe)[0] != want_total;
        errors += fetch(partial, 1, pe)[0] != kInputs * (pe + 1 - kCorrection);
    }
    HIP_CHECK(hipStreamDestroy(stream));
    nvshmem_free(input), nvshmem_free(partial), nvshmem_free(total);
    return finish("on_stream", errors);
}
