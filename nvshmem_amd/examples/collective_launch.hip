// A value travels around the ring npes times and every PE adds its rank on each pass, the kernel of
// the reference's examples/collective-launch.cu:32-44: nvshmem_int_p to the right neighbour, then two
// barriers per step inside the kernel - which is why it needs nvshmemx_collective_launch (all PEs'
// blocks have to be resident at the same time).  Closed form: PE p starts with p and after n steps
// holds p + (p-1) + ... + (p-n) with the indices mod n, that is n (n-1) / 2 + p.
#include "example_util.hpp"

__global__ void reduce_ring(int *target) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    const int peer = (me + 1) % np;
    int *mine = (int *)nvshmem_ptr(target, me);
    int value = me;
    for (int i = 0; i < np; ++i) {
        nvshmem_int_p(target, value, peer);
        nvshmem_barrier_all();
        value = *(volatile int *)mine + me;
        nvshmem_barrier_all();
    }
    *mine = value;
}

int main() {
    nvshmem_init();
    const int np = nvshmem_n_pes();
    int *target = (int *)nvshmem_calloc(1, sizeof(int));
    int grid = 0;
    NVSHMEM_CHECK(nvshmemx_collective_launch_query_gridsize((const void *)reduce_ring, dim3(1), nullptr, 0, &grid));
    long errors = grid < 1;
    void *args[] = {&target};
    NVSHMEM_CHECK(nvshmemx_collective_launch((const void *)reduce_ring, dim3(1), dim3(1), args, 0, nullptr));
    HIP_CHECK(hipDeviceSynchronize());
    for (int pe = 0; pe < np; ++pe) errors += fetch(target, 1, pe)[0] != np * (np - 1) / 2 + pe;
    nvshmem_free(target);
    return finish("collective_launch", errors);
}
