// The token dispatch that signals every row: one nvshmemx_putmem_signal_nbi per row copy, the form
// the reference's signalling idiom takes (examples/ring-reduce.cu:111-127) on the token shuffle of
// examples/moe_shuffle.cu:240-289.  A translation unit of its own because of its copy depth: a row of
// 14336 bytes is 14 vectors per lane of a wavefront, and with rounds of 14 a put is one run of loads
// followed by one run of stores (4.53 -> 4.90 TB/s against rounds of 8 + 4 + 2); the 56 vector
// registers that costs would take occupancy from the one-wavefront blocks of the other shuffle kernels.
#include <hip/hip_runtime.h>

#define NVSHMEMI_AMD_COPY_UNROLL 14

#include "nvshmem_perftest.h"
#include "nvshmemx.h"
#include "moe_common.hpp"
#include "perftest_common.hpp"

namespace {

// Per-row signalling: the API-literal form, one nvshmemx_putmem_signal_nbi per row.
template <bool WARP_SCOPED>
__global__ void moe_dispatch_rowsignal_kernel(char *recv, const char *send, const int32_t *dest_pe,
                                              const int64_t *dest_row, const uint64_t *expected,
                                              uint64_t *sig, int tokens, int topk,
                                              size_t row_bytes, size_t recv_cap_rows, int sig_op,
                                              int sig_stride) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    const int32_t *my_dest_pe = (const int32_t *)nvshmem_ptr(dest_pe, me);
    const int64_t *my_dest_row = (const int64_t *)nvshmem_ptr(dest_row, me);
    const size_t rows = (size_t)tokens * (size_t)topk;
    if (WARP_SCOPED) {
        const size_t waves_per_block = blockDim.x / NVSHMEMI_WARP_SIZE;
        const size_t wave = blockIdx.x * waves_per_block + wave_in_block();
        const size_t nwaves = (size_t)gridDim.x * waves_per_block;
        // Up to four consecutive wavefronts of a block share a token and send a quarter of its topk copies each,
        // one behind the other: the token's row is fetched from memory once, by whichever of them comes first,
        // and every other read of it hits in this XCD's L2.  (A wavefront that sent all topk copies of its own
        // token re-read the row seven times while 255 other wavefronts of the XCD streamed their rows through the
        // same 4 MiB: about one re-read in seven missed - measured traffic 1.13 times the algorithmic bytes, 1.00
        // with the sharing, at the same or a slightly better rate.)
        unsigned share = 1;
        while (share < 4 && waves_per_block % (2 * share) == 0 && topk % (int)(2 * share) == 0) share *= 2;
        const int per = topk / (int)share;
        for (size_t u = wave; u < (size_t)tokens * share; u += nwaves) {
            const size_t t = u / share;
            const int k0 = (int)(u % share) * per;
            for (int k = k0; k < k0 + per; ++k) {
                const size_t r = t * (size_t)topk + (size_t)k;
                if (row_ok(my_dest_pe[r], my_dest_row[r], np, recv_cap_rows))
                    nvshmemx_putmem_signal_nbi_warp(recv + (size_t)my_dest_row[r] * row_bytes,
                                                    send + t * row_bytes, row_bytes,
                                                    sig + (size_t)me * sig_stride, 1, sig_op, my_dest_pe[r]);
            }
        }
    } else {
        for (size_t r = blockIdx.x; r < rows; r += gridDim.x)
            if (row_ok(my_dest_pe[r], my_dest_row[r], np, recv_cap_rows))
            nvshmemx_putmem_signal_nbi_block(recv + (size_t)my_dest_row[r] * row_bytes,
                                             send + (r / (size_t)topk) * row_bytes, row_bytes,
                                             sig + (size_t)me * sig_stride, 1, sig_op, my_dest_pe[r]);
    }
    if (blockIdx.x == 0) {
        const uint64_t *my_expected = (const uint64_t *)nvshmem_ptr(expected, me);
        for (int src = threadIdx.x; src < np; src += blockDim.x)
            nvshmem_signal_wait_until(sig + (size_t)src * sig_stride, NVSHMEM_CMP_GE, my_expected[src]);
    }
}

}  // namespace

namespace perftest {

int launch_moe_rowsignal(bool warp, int blocks_per_pe, int threads, void **args, hipStream_t stream) {
    const void *fn = warp ? (const void *)moe_dispatch_rowsignal_kernel<true>
                          : (const void *)moe_dispatch_rowsignal_kernel<false>;
    return nvshmemx_collective_launch(fn, dim3(blocks_per_pe), dim3(threads), args, 0, stream);
}

}  // namespace perftest
