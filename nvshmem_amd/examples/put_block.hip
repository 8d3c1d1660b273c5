// Ring shift with a block-scoped put, the workload of the reference's examples/put-block.cu: every PE
// pushes a vector filled with its own number to its right neighbour, so PE p must end up holding
// (p - 1 + npes) % npes in every element (the reference's check, put-block.cu:93-104).
#include "example_util.hpp"

__global__ void shift_right(int *recv, int *send, size_t n) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    // each block owns a contiguous slice of the vector
    const size_t per_block = n / gridDim.x, at = blockIdx.x * per_block;
    int *mine = (int *)nvshmem_ptr(send, me);
    for (size_t i = threadIdx.x; i < per_block; i += blockDim.x) mine[at + i] = me;
    __syncthreads();
    nvshmemx_int_put_block(recv + at, send + at, per_block, (me + 1) % np);
}

int main() {
    nvshmem_init();
    const int np = nvshmem_n_pes();
    const size_t n = 1 << 20;
    int *send = (int *)nvshmem_malloc(n * sizeof(int));
    int *recv = (int *)nvshmem_calloc(n, sizeof(int));
    void *args[] = {&recv, &send, (void *)&n};
    NVSHMEM_CHECK(nvshmemx_collective_launch((const void *)shift_right, dim3(32), dim3(256), args, 0, nullptr));
    nvshmem_barrier_all();
    long errors = 0;
    for (int pe = 0; pe < np; ++pe)
        for (int v : fetch(recv, n, pe)) errors += v != (pe - 1 + np) % np;
    nvshmem_free(send);
    nvshmem_free(recv);
    return finish("put_block", errors);
}
