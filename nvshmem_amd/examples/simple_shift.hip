// The first program of the reference's programming guide (examples/dev-guide-ring.cu:15-45): every PE
// writes its rank into its right neighbour's copy of one symmetric int with nvshmem_int_p from a
// one-thread kernel on a stream, a barrier on the same stream completes the transfer, and the host
// reads the message back: PE p must have received (p - 1 + npes) % npes.
#include "example_util.hpp"

__global__ void simple_shift(int *destination) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    nvshmem_int_p(destination, me, (me + 1) % np);
}

int main() {
    nvshmem_init();
    const int np = nvshmem_n_pes();
    hipStream_t stream;
    HIP_CHECK(hipStreamCreate(&stream));
    int *destination = (int *)nvshmem_malloc(sizeof(int));
    // one block per logical PE: the third grid dimension stands where the reference has one process each
    hipLaunchKernelGGL(simple_shift, dim3(1, 1, np), dim3(1), 0, stream, destination);
    HIP_CHECK(hipGetLastError());
    nvshmemx_barrier_all_on_stream(stream);
    long errors = 0;
    for (int pe = 0; pe < np; ++pe) {
        int msg = -1;
        HIP_CHECK(hipMemcpyAsync(&msg, nvshmem_ptr(destination, pe), sizeof(int), hipMemcpyDeviceToHost, stream));
        HIP_CHECK(hipStreamSynchronize(stream));
        printf("%d: received message %d\n", pe, msg);
        errors += msg != (pe - 1 + np) % np;
    }
    nvshmem_free(destination);
    HIP_CHECK(hipStreamDestroy(stream));
    return finish("simple_shift", errors);
}
