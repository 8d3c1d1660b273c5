// Broadcast around a ring, the pattern of the reference's examples/ring-bcast.cu: PE 0 owns the data,
// every other PE waits until its left neighbour has delivered it and passes it on.  The payload and
// the "it has arrived" flag travel together in one put-with-signal.  Known answer of the reference
// (ring-bcast.cu:44-72): PE 0 starts with data[i] = i, everybody ends with data[i] = i.
#include "example_util.hpp"

__global__ void ring_bcast(int *data, size_t n, uint64_t *arrived) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    if (me != 0) {
        if (threadIdx.x == 0) nvshmem_signal_wait_until(arrived, NVSHMEM_CMP_EQ, 1);
        __syncthreads();
    }
    if (me != np - 1)
        nvshmemx_int_put_signal_block(data, data, n, arrived, 1, NVSHMEM_SIGNAL_SET, me + 1);
}

int main() {
    nvshmem_init();
    const int np = nvshmem_n_pes();
    const size_t n = 4096;
    int *data = (int *)nvshmem_malloc(n * sizeof(int));
    uint64_t *arrived = (uint64_t *)nvshmem_calloc(1, sizeof(uint64_t));
    for (int pe = 0; pe < np; ++pe) {
        std::vector<int> init(n);
        for (size_t i = 0; i < n; ++i) init[i] = pe == 0 ? (int)i : -1;
        store(data, init, pe);
    }
    void *args[] = {&data, (void *)&n, &arrived};
    NVSHMEM_CHECK(nvshmemx_collective_launch((const void *)ring_bcast, dim3(1), dim3(256), args, 0, nullptr));
    nvshmem_barrier_all();
    long errors = 0;
    for (int pe = 0; pe < np; ++pe) {
        const std::vector<int> got = fetch(data, n, pe);
        for (size_t i = 0; i < n; ++i) errors += got[i] != (int)i;
    }
    nvshmem_free(data);
    nvshmem_free(arrived);
    return finish("ring_bcast", errors);
}
