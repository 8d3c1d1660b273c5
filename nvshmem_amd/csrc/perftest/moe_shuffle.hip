// MoE token shuffle on logical PEs: dispatch rows to the PEs that own their experts with
// put + signal, wait for the expected row counts, and combine (gather the rows back).
//
// Workload model: examples/moe_shuffle.cu in the reference tree (offset exchange :204-234, one row
// per thread group pushed to `expert / experts_per_pe` :240-289); the signalling idiom is the
// put_signal_nbi + signal_wait_until(GE) pair of examples/ring-reduce.cu:111-127.
//
// A row of 14336 bytes is 896 16-byte vectors: a wavefront moves it with 14 vectors per lane, so
// the default scope is one row per wavefront with no block-wide synchronisation in the loop.
#include <hip/hip_runtime.h>
#include <atomic>
#include <cstdlib>
#include <mutex>

// A row is 14 vectors per lane: rounds of 8 + 4 + 2 keep more loads in flight than the default
// 4 + 4 + 4 + 2 (measured 5 % faster for dispatch and combine).  (The kernel that signals every row is
// built with rounds of 14 in a translation unit of its own, moe_rowsignal.hip.)
#define NVSHMEMI_AMD_COPY_UNROLL 8

#include "nvshmem_perftest.h"
#include "nvshmemx.h"
#include "moe_common.hpp"
#include "perftest_common.hpp"

// Signal words of the dispatch that allocates nothing (nvshmem_perftest_moe_dispatch_pieces_static):
// kStaticSignalPes rows of kStaticSignalPes words, 8 KiB.  Device memory of this code object: every GPU
// the library runs on holds its own copy, at its own address, until the process ends.  In host code the
// name is only a handle for hipGetSymbolAddress; kernels get the address that call returns.
constexpr int kStaticSignalPes = 32;
static __device__ __align__(256) uint64_t scratch[kStaticSignalPes * kStaticSignalPes];

namespace {

constexpr int kMaxPes = NVSHMEMI_AMD_MAX_PES;

// Dispatch.  Rows are dealt round-robin to the thread groups of the PE's blocks.  Each group tallies
// what it sent to every destination; once all its puts are complete it adds the tallies to the
// destinations' signal words (one release + npes atomic adds per block instead of one per row).
template <bool WARP_SCOPED>
__global__ void moe_dispatch_kernel(char *recv, const char *send, const int32_t *dest_pe,
                                    const int64_t *dest_row, const uint64_t *expected,
                                    uint64_t *sig, int tokens, int topk, size_t row_bytes,
                                    size_t recv_cap_rows) {
    __shared__ unsigned tally[kMaxPes];
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    const int32_t *my_dest_pe = (const int32_t *)nvshmem_ptr(dest_pe, me);
    const int64_t *my_dest_row = (const int64_t *)nvshmem_ptr(dest_row, me);
    const size_t rows = (size_t)tokens * (size_t)topk;
    for (int i = threadIdx.x; i < np; i += blockDim.x) tally[i] = 0;
    __syncthreads();

    if (WARP_SCOPED) {
        const size_t waves_per_block = blockDim.x / NVSHMEMI_WARP_SIZE;
        const size_t wave = blockIdx.x * waves_per_block + wave_in_block_per_lane();
        const size_t nwaves = (size_t)gridDim.x * waves_per_block;
        const bool lane0 = (threadIdx.x % NVSHMEMI_WARP_SIZE) == 0;
        // A wavefront takes a token and pushes its topk copies back to back: the first put streams
        // the row from HBM, the others find it in this XCD's L2, so every source row crosses the HBM
        // interface once and is written topk times.
        for (size_t t = wave; t < (size_t)tokens; t += nwaves) {
            const char *src_row = send + t * row_bytes;
            for (int k = 0; k < topk; ++k) {
                const size_t r = t * (size_t)topk + (size_t)k;
                const int pe = my_dest_pe[r];
                const int64_t row = my_dest_row[r];
                if (!row_ok(pe, row, np, recv_cap_rows)) continue;
                nvshmemx_putmem_nbi_warp(recv + (size_t)row * row_bytes, src_row, row_bytes, pe);
                if (lane0) atomicAdd(&tally[pe], 1u);
            }
        }
    } else {
        for (size_t r = blockIdx.x; r < rows; r += gridDim.x) {
            const int pe = my_dest_pe[r];
            if (!row_ok(pe, my_dest_row[r], np, recv_cap_rows)) continue;
            nvshmemx_putmem_nbi_block(recv + (size_t)my_dest_row[r] * row_bytes,
                                      send + (r / (size_t)topk) * row_bytes, row_bytes, pe);
            if (threadIdx.x == 0) tally[pe] += 1u;
        }
    }
    // all rows of this block are written; publish the counts
    nvshmemx_quiet_block();
    for (int pe = threadIdx.x; pe < np; pe += blockDim.x)
        if (tally[pe]) nvshmemx_signal_op(sig + me, (uint64_t)tally[pe], NVSHMEM_SIGNAL_ADD, pe);

    // receiver side: block 0 of every PE waits until each source has delivered what it announced
    if (blockIdx.x == 0) {
        const uint64_t *my_expected = (const uint64_t *)nvshmem_ptr(expected, me);
        for (int src = threadIdx.x; src < np; src += blockDim.x)
            nvshmem_signal_wait_until(sig + src, NVSHMEM_CMP_GE, my_expected[src]);
    }
}

// Dispatch cut into short work items: an item is one piece of one token's row, pushed to all of the
// token's topk destinations by one wavefront.  Grid: blockIdx.x = piece of the row, blockIdx.y (times
// the wavefronts of a block) = token, so neither needs a division and consecutive blocks work on the
// same row.  No tallies and no signalling here: the counts are published by
// moe_dispatch_signal_kernel, launched behind this kernel on the same stream, so the end of this
// kernel is what orders every row before its signal.
//
// PIECE bytes per item, moved with nvshmemx_putmem_nbi_warp (any alignment, any row size): the first
// put streams the piece from HBM, the others find it in the cache.
template <int PIECE>
__global__ void moe_dispatch_pieces_kernel(char *recv, const char *send, const int32_t *dest_pe,
                                           const int64_t *dest_row, int tokens, int topk,
                                           size_t row_bytes, size_t recv_cap_rows) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    const int32_t *my_dest_pe = (const int32_t *)nvshmem_ptr(dest_pe, me);
    const int64_t *my_dest_row = (const int64_t *)nvshmem_ptr(dest_row, me);
    const unsigned waves_per_block = blockDim.x / NVSHMEMI_WARP_SIZE;
    const size_t off = (size_t)blockIdx.x * PIECE;
    if (off >= row_bytes) return;
    const size_t len = row_bytes - off < (size_t)PIECE ? row_bytes - off : (size_t)PIECE;
    for (size_t t = (size_t)blockIdx.y * waves_per_block + wave_in_block(); t < (size_t)tokens;
         t += (size_t)gridDim.y * waves_per_block) {
        const char *src = send + t * row_bytes + off;
        for (int k = 0; k < topk; ++k) {
            const size_t r = t * (size_t)topk + (size_t)k;
            const int pe = my_dest_pe[r];
            const int64_t row = my_dest_row[r];
            if (!row_ok(pe, row, np, recv_cap_rows)) continue;
            nvshmemx_putmem_nbi_warp(recv + (size_t)row * row_bytes + off, src, len, pe);
        }
    }
}

// The same work items moved with nvshmem_ptr and plain vector accesses: the piece is loaded into
// registers (V 16-byte vectors per lane) and stored to up to four of the topk destinations from there;
// the blocks that share a piece are neighbours in the grid; they run on different XCDs, so the second
// one's load is served by the Infinity Cache rather than by L2 (measured: FETCH_SIZE 1840 MiB for
// 896 MiB of rows), and a source byte still crosses the HBM interface once instead of topk times.
// Sharers placed on one XCD hit in L2 (FETCH_SIZE 944 MiB) but the kernel is 11 % slower.  Needs 16-byte aligned buffers and
// rows; the host picks moe_dispatch_pieces_kernel otherwise.
template <int V>
__global__ void moe_dispatch_direct_kernel(char *recv, const char *send, const int32_t *dest_pe,
                                           const int64_t *dest_row, int tokens, int topk,
                                           size_t row_bytes, size_t recv_cap_rows, unsigned kshift) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    const int32_t *my_dest_pe = (const int32_t *)nvshmem_ptr(dest_pe, me);
    const int64_t *my_dest_row = (const int64_t *)nvshmem_ptr(dest_row, me);
    const nvshmemi_v4u *my_send = (const nvshmemi_v4u *)nvshmem_ptr(send, me);
    const unsigned waves_per_block = blockDim.x / NVSHMEMI_WARP_SIZE;
    const unsigned row_vecs = (unsigned)(row_bytes / 16);
    const unsigned v0 = (blockIdx.x >> kshift) * (64 * V) + threadIdx.x % NVSHMEMI_WARP_SIZE;
    // 2^kshift neighbouring blocks share a piece and split the token's copies between them
    const int kper = (topk + (1 << kshift) - 1) >> kshift;
    const int k0 = (int)(blockIdx.x & ((1u << kshift) - 1)) * kper;
    const int k1 = k0 + kper < topk ? k0 + kper : topk;
    for (size_t t = (size_t)blockIdx.y * waves_per_block + wave_in_block(); t < (size_t)tokens;
         t += (size_t)gridDim.y * waves_per_block) {
        const nvshmemi_v4u *src = my_send + t * row_vecs;
        nvshmemi_v4u x[V];
#pragma unroll
        for (int u = 0; u < V; ++u)
            if (v0 + 64 * u < row_vecs) x[u] = kshift ? src[v0 + 64 * u] : __builtin_nontemporal_load(src + v0 + 64 * u);
        for (int k = k0; k < k1; ++k) {
            const size_t r = t * (size_t)topk + (size_t)k;
            const int pe = my_dest_pe[r];
            const int64_t row = my_dest_row[r];
            if (!row_ok(pe, row, np, recv_cap_rows)) continue;
            nvshmemi_v4u *d = (nvshmemi_v4u *)nvshmem_ptr(recv, pe) + (size_t)row * row_vecs;
#pragma unroll
            for (int u = 0; u < V; ++u)
                if (v0 + 64 * u < row_vecs) __builtin_nontemporal_store(x[u], d + v0 + 64 * u);
        }
    }
}

// A few blocks per PE: each counts the rows of its share that this PE sent to every destination and
// adds the counts to the destinations' signal words; block 0 then waits until every source has
// announced what this PE expects.
// SYMMETRIC: `sig` is a symmetric array of npes words per PE, updated with nvshmemx_signal_op.  Otherwise
// it is an ordinary device array of npes rows of npes words (row p = the signal words of PE p), which
// the symmetric-address API cannot name, so the words are updated with the same agent-scope add directly.
template <bool SYMMETRIC>
__global__ void moe_dispatch_signal_kernel(const int32_t *dest_pe, const int64_t *dest_row,
                                           const uint64_t *expected, uint64_t *sig, int tokens,
                                           int topk, size_t recv_cap_rows) {
    __shared__ unsigned tally[kMaxPes];
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    const int32_t *my_dest_pe = (const int32_t *)nvshmem_ptr(dest_pe, me);
    const int64_t *my_dest_row = (const int64_t *)nvshmem_ptr(dest_row, me);
    const size_t rows = (size_t)tokens * (size_t)topk;
    for (int i = threadIdx.x; i < np; i += blockDim.x) tally[i] = 0;
    __syncthreads();
    // Eight routing entries per thread are fetched before the first is counted (one after the other
    // every entry paid the way to memory), and the counting stays in registers: lane l of a wavefront
    // answers for destination l (np <= 64) and learns the other lanes' destinations by ballots.  An
    // atomicAdd per row into np shared words serialised the 1024 threads: 65536 rows took 62 us, with
    // the batched loads alone 47 us.
    const unsigned lane = threadIdx.x % NVSHMEMI_WARP_SIZE;
    unsigned mine = 0;
    // the blocks of a PE share the rows; every block announces its own counts (the signals add up)
    for (size_t r0 = (size_t)blockIdx.x * blockDim.x + threadIdx.x - lane; r0 < rows;
         r0 += 8 * (size_t)blockDim.x * gridDim.x) {  // wave-uniform trip count
        int to[8];
        int64_t row[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const size_t r = r0 + lane + (size_t)k * blockDim.x * gridDim.x;
            const size_t rc = r < rows ? r : rows - 1;
            to[k] = my_dest_pe[rc];
            row[k] = my_dest_row[rc];
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const size_t r = r0 + lane + (size_t)k * blockDim.x * gridDim.x;
            const int dest = r < rows && row_ok(to[k], row[k], np, recv_cap_rows) ? to[k] : -1;
            for (int pe = 0; pe < np; ++pe) {
                const unsigned c = (unsigned)__builtin_popcountll(__builtin_amdgcn_ballot_w64(dest == pe));
                if ((int)lane == pe) mine += c;
            }
        }
    }
    if ((int)lane < np && mine) atomicAdd(&tally[lane], mine);
    __syncthreads();
    for (int pe = threadIdx.x; pe < np; pe += blockDim.x)
        if (tally[pe]) {
            if (SYMMETRIC) nvshmemx_signal_op(sig + me, (uint64_t)tally[pe], NVSHMEM_SIGNAL_ADD, pe);
            else __hip_atomic_fetch_add(sig + (size_t)pe * np + me, (uint64_t)tally[pe], __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
        }
    if (blockIdx.x != 0) return;
    const uint64_t *my_expected = (const uint64_t *)nvshmem_ptr(expected, me);
    // (an address outside the symmetric heap is waited on as it is)
    uint64_t *my_words = SYMMETRIC ? sig : sig + (size_t)me * np;
    for (int src = threadIdx.x; src < np; src += blockDim.x)
        nvshmem_signal_wait_until(my_words + src, NVSHMEM_CMP_GE, my_expected[src]);
}

// PIECE > 0 (wavefront scope): a work item is PIECE bytes of a row instead of a whole row, so that
// with one wavefront per block every block moves one short aligned piece and exits.
template <bool WARP_SCOPED, int PIECE = 0>
__global__ void moe_combine_kernel(char *out, const char *recv, const int32_t *dest_pe,
                                   const int64_t *dest_row, int tokens, int topk,
                                   size_t row_bytes, size_t recv_cap_rows) {
    const int me = nvshmem_my_pe();
    const int np = nvshmem_n_pes();
    const int32_t *my_dest_pe = (const int32_t *)nvshmem_ptr(dest_pe, me);
    const int64_t *my_dest_row = (const int64_t *)nvshmem_ptr(dest_row, me);
    const size_t rows = (size_t)tokens * (size_t)topk;
    if (WARP_SCOPED) {
        const size_t waves_per_block = blockDim.x / NVSHMEMI_WARP_SIZE;
        const size_t wave = blockIdx.x * waves_per_block + wave_in_block();
        const size_t nwaves = (size_t)gridDim.x * waves_per_block;
        if (PIECE > 0) {
            // (the item index is wave-uniform and, as the host entry point checks, below 2^32: a scalar
            // 32-bit division instead of a 64-bit one per lane, which took some 40 vector registers)
            const uint32_t pieces = (uint32_t)((row_bytes + PIECE - 1) / PIECE);
            const uint32_t items = (uint32_t)rows * pieces;
            for (uint32_t item = (uint32_t)wave; item < items; item += (uint32_t)nwaves) {
                const size_t r = item / pieces, off = (size_t)(item - (uint32_t)r * pieces) * PIECE;
                const size_t len = row_bytes - off < (size_t)PIECE ? row_bytes - off : (size_t)PIECE;
                __builtin_assume(len <= (size_t)PIECE);   // short copies: the engine's long-copy code drops out
                if (row_ok(my_dest_pe[r], my_dest_row[r], np, recv_cap_rows))
                    nvshmemx_getmem_nbi_warp(out + r * row_bytes + off,
                                             recv + (size_t)my_dest_row[r] * row_bytes + off, len,
                                             my_dest_pe[r]);
            }
            return;
        }
        for (size_t r = wave; r < rows; r += nwaves)
            if (row_ok(my_dest_pe[r], my_dest_row[r], np, recv_cap_rows))
            nvshmemx_getmem_nbi_warp(out + r * row_bytes, recv + (size_t)my_dest_row[r] * row_bytes,
                                     row_bytes, my_dest_pe[r]);
    } else {
        for (size_t r = blockIdx.x; r < rows; r += gridDim.x)
            if (row_ok(my_dest_pe[r], my_dest_row[r], np, recv_cap_rows))
            nvshmemx_getmem_nbi_block(out + r * row_bytes, recv + (size_t)my_dest_row[r] * row_bytes,
                                      row_bytes, my_dest_pe[r]);
    }
}

// counts exchange + prefix sums: every PE fetches all PEs' per-expert counts with scalar gets and
// lays out the receive segments of every destination PE in (expert, source PE) order.
__global__ void moe_exchange_offsets_kernel(const int64_t *counts, int64_t *seg_base,
                                            int64_t *recv_rows, int num_experts) {
    extern __shared__ int64_t table[];  // [expert][src]
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    const int epp = num_experts / np;
    for (int i = threadIdx.x; i < num_experts * np; i += blockDim.x)
        table[i] = nvshmem_int64_g(counts + i / np, i % np);
    __syncthreads();
    int64_t *my_seg = (int64_t *)nvshmem_ptr(seg_base, me);
    for (int d = threadIdx.x; d < np; d += blockDim.x) {
        int64_t run = 0;
        for (int i = d * epp * np; i < (d + 1) * epp * np; ++i) {
            my_seg[i] = run;
            run += table[i];
        }
        if (d == me) ((int64_t *)nvshmem_ptr(recv_rows, me))[0] = run;
    }
}

__global__ void clear_words_kernel(uint64_t *words, unsigned n) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) words[i] = 0;
}

// Address of this device's copy of `scratch`.  The lookup (hipGetSymbolAddress: a runtime call that may load
// the code object) happens once per device, under a lock, in nvshmem_perftest_static_init or in the first
// call of the entry point on that device - never under stream capture: `may_lookup` is false there, and an
// address that is not known yet is then an error.
constexpr int kMaxDevices = 64;
std::mutex scratch_lock;
uint64_t *scratch_ptr[kMaxDevices];
std::atomic<int> scratch_calls_in_progress[kMaxDevices];   // host threads inside the entry point, per device

int current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        fprintf(stderr, "nvshmem_perftest: no current device for the static signal words\n");
        return -1;
    }
    return dev;
}

uint64_t *scratch_address(int dev, bool may_lookup) {
    std::lock_guard<std::mutex> lock(scratch_lock);
    if (!scratch_ptr[dev]) {
        if (!may_lookup) {
            fprintf(stderr, "nvshmem_perftest: the static signal words of device %d are not looked up yet and the "
                            "stream is being captured; call nvshmem_perftest_static_init() first\n", dev);
            return nullptr;
        }
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            fprintf(stderr, "nvshmem_perftest: hipGetSymbolAddress(scratch) failed: %s\n", hipGetErrorString(e));
            return nullptr;
        }
        scratch_ptr[dev] = (uint64_t *)p;
    }
    return scratch_ptr[dev];
}

bool moe_args_ok(const void *table_pe, const void *table_row, int tokens, int topk,
                 size_t row_bytes, int blocks, int threads, bool warp) {
    if (!perftest::ready() || tokens < 1 || topk < 1 || row_bytes == 0 ||
        !perftest::check_launch(blocks, threads))
        return false;
    if (warp && (threads % NVSHMEMI_WARP_SIZE)) {
        fprintf(stderr, "nvshmem_perftest: warp-scoped shuffle needs a multiple of 64 threads\n");
        return false;
    }
    const size_t rows = (size_t)tokens * (size_t)topk;
    return perftest::check_range(table_pe, rows * sizeof(int32_t)) &&
           perftest::check_range(table_row, rows * sizeof(int64_t));
}

}  // namespace

extern "C" {

// scope: NVSHMEM_PERFTEST_SCOPE_WARP (row per wavefront) or _BLOCK (row per block);
// bit 8 set (scope | 256) selects per-row signalling instead of per-block tallies, bit 9 (| 512) with
// it the NVSHMEMX_AMD_SIGNAL_PAYLOAD_ONLY ordering of those signals.  The signal word of source PE s
// is sig[s * sig_stride] (per-row signalling only; the tallies use stride 1).
int nvshmem_perftest_moe_dispatch_put_signal(void *recv, size_t recv_cap_rows, const void *send,
                                             const int32_t *dest_pe, const int64_t *dest_row,
                                             const uint64_t *expected, uint64_t *sig, int sig_stride,
                                             int tokens, int topk, size_t row_bytes, int blocks_per_pe,
                                             int threads, int scope, void *stream) {
    const bool per_row = (scope & 256) != 0;
    int sig_op = NVSHMEM_SIGNAL_ADD | ((scope & 512) ? NVSHMEMX_AMD_SIGNAL_PAYLOAD_ONLY : 0);
    const bool warp = (scope & 255) == NVSHMEM_PERFTEST_SCOPE_WARP;
    if (!warp && (scope & 255) != NVSHMEM_PERFTEST_SCOPE_BLOCK) return NVSHMEMX_ERROR_INVALID_VALUE;
    if (sig_stride < 1 || (!per_row && sig_stride != 1)) return NVSHMEMX_ERROR_INVALID_VALUE;
    if (!moe_args_ok(dest_pe, dest_row, tokens, topk, row_bytes, blocks_per_pe, threads, warp))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    const size_t words = sizeof(uint64_t) * (size_t)nvshmem_n_pes();
    if (!perftest::check_range(expected, words) || !perftest::check_range(sig, words * (size_t)sig_stride) ||
        !perftest::check_range(send, (size_t)tokens * row_bytes) ||
        !perftest::check_range(recv, recv_cap_rows * row_bytes))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    char *r = (char *)recv;
    const char *s = (const char *)send;
    void *args[] = {&r, &s, &dest_pe, &dest_row, &expected, &sig, &tokens, &topk, &row_bytes,
                    &recv_cap_rows, &sig_op, &sig_stride};
    if (per_row) return perftest::launch_moe_rowsignal(warp, blocks_per_pe, threads, args, (hipStream_t)stream);
    const void *fn = warp ? (const void *)moe_dispatch_kernel<true> : (const void *)moe_dispatch_kernel<false>;
    return nvshmemx_collective_launch(fn, dim3(blocks_per_pe), dim3(threads), args, 0,
                                      (hipStream_t)stream);
}

int nvshmem_perftest_moe_dispatch_ex(void *recv, size_t recv_cap_rows, const void *send, const int32_t *dest_pe,
                                     const int64_t *dest_row, const uint64_t *expected,
                                     uint64_t *sig, int tokens, int topk, size_t row_bytes,
                                     int blocks_per_pe, int threads, int scope, void *stream) {
    return nvshmem_perftest_moe_dispatch_put_signal(recv, recv_cap_rows, send, dest_pe, dest_row, expected, sig,
                                                    1, tokens, topk, row_bytes, blocks_per_pe, threads, scope,
                                                    stream);
}

int nvshmem_perftest_moe_dispatch(void *recv, size_t recv_cap_rows, const void *send, const int32_t *dest_pe,
                                  const int64_t *dest_row, const uint64_t *expected, uint64_t *sig,
                                  int tokens, int topk, size_t row_bytes, int blocks_per_pe,
                                  int threads, void *stream) {
    return nvshmem_perftest_moe_dispatch_ex(recv, recv_cap_rows, send, dest_pe, dest_row, expected, sig, tokens,
                                            topk, row_bytes, blocks_per_pe, threads,
                                            NVSHMEM_PERFTEST_SCOPE_WARP, stream);
}

// Dispatch as two launches on `stream`: a grid with one wavefront per work item - piece_bytes (1024 /
// 2048 / 4096) of a token's row, pushed to its topk destinations - then one block per PE that
// publishes the row counts through the signal words and waits for the expected ones.  `threads` (a
// multiple of 64) sets how many tokens a block takes.
// static_sig: the signal words are this device's `scratch` rows (cleared here, on the stream, by a
// kernel) instead of the caller's symmetric array.
static int dispatch_pieces(void *recv, size_t recv_cap_rows, const void *send, const int32_t *dest_pe,
                           const int64_t *dest_row, const uint64_t *expected, uint64_t *sig,
                           uint64_t *static_sig, int tokens, int topk, size_t row_bytes, int piece_bytes,
                           int threads, void *stream) {
    if (piece_bytes != 1024 && piece_bytes != 2048 && piece_bytes != 4096) return NVSHMEMX_ERROR_INVALID_VALUE;
    if (!moe_args_ok(dest_pe, dest_row, tokens, topk, row_bytes, 1, threads, true))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    const size_t words = sizeof(uint64_t) * (size_t)nvshmem_n_pes();
    const size_t pieces = (row_bytes + (size_t)piece_bytes - 1) / (size_t)piece_bytes;
    if (pieces > 0x7fffffffull || !perftest::check_range(expected, words) ||
        (!static_sig && !perftest::check_range(sig, words)) ||
        !perftest::check_range(send, (size_t)tokens * row_bytes) ||
        !perftest::check_range(recv, recv_cap_rows * row_bytes))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    const unsigned waves = (unsigned)threads / NVSHMEMI_WARP_SIZE;
    unsigned token_blocks = ((unsigned)tokens + waves - 1) / waves;
    if (token_blocks > 65535u) token_blocks = 65535u;  // the kernels stride over the rest
    const dim3 grid((unsigned)pieces, token_blocks, (unsigned)nvshmem_n_pes());
    const bool aligned = row_bytes % 16 == 0 && ((uintptr_t)recv | (uintptr_t)send) % 16 == 0;
    const bool direct = aligned && getenv("NVSHMEM_PERFTEST_MOE_PUTS") == nullptr;
    // at most four copies per wavefront (measured 1.62 -> 1.56 ms for top-8; two per wavefront is slower)
    unsigned kshift = 0;
    while (((topk + (1 << kshift) - 1) >> kshift) > 4) ++kshift;
    const dim3 dgrid(grid.x << kshift, grid.y, grid.z);
    if (static_sig) {
        const unsigned n = (unsigned)(nvshmem_n_pes() * nvshmem_n_pes());
        hipLaunchKernelGGL(clear_words_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, static_sig, n);
        const int rc0 = perftest::launch_status("clear_words");
        if (rc0 != 0) return rc0;
    }
#define LAUNCH_DIRECT(V)                                                                           \
    hipLaunchKernelGGL((moe_dispatch_direct_kernel<V>), dgrid, dim3(threads), 0, (hipStream_t)stream, \
                       (char *)recv, (const char *)send, dest_pe, dest_row, tokens, topk, row_bytes, \
                       recv_cap_rows, kshift)
#define LAUNCH_DISPATCH(P)                                                                         \
    hipLaunchKernelGGL((moe_dispatch_pieces_kernel<P>), grid, dim3(threads), 0, (hipStream_t)stream, \
                       (char *)recv, (const char *)send, dest_pe, dest_row, tokens, topk, row_bytes, \
                       recv_cap_rows)
    if (direct) {
        if (piece_bytes == 1024) LAUNCH_DIRECT(1);
        else if (piece_bytes == 2048) LAUNCH_DIRECT(2);
        else LAUNCH_DIRECT(4);
    } else if (piece_bytes == 1024) LAUNCH_DISPATCH(1024);
    else if (piece_bytes == 2048) LAUNCH_DISPATCH(2048);
    else LAUNCH_DISPATCH(4096);
#undef LAUNCH_DISPATCH
#undef LAUNCH_DIRECT
    int rc = perftest::launch_status("moe_dispatch_pieces");
    if (rc != 0) return rc;
    // one block per PE scanning alone is bound by its own memory latency (65536 rows: 46 us); with a
    // few blocks per PE the scan is short.  An ordinary launch is enough: a block announces its counts
    // before it waits and only block 0 of each PE waits at all, so the blocks that wait (one per PE, at
    // most 64) can never keep a block that still has to announce off the GPU
    const unsigned sig_blocks = (unsigned)(((size_t)tokens * (size_t)topk + 8191) / 8192 < 8 ? ((size_t)tokens * (size_t)topk + 8191) / 8192 : 8);
    if (static_sig)
        hipLaunchKernelGGL(moe_dispatch_signal_kernel<false>, dim3(sig_blocks, 1, (unsigned)nvshmem_n_pes()), dim3(1024),
                           0, (hipStream_t)stream, dest_pe, dest_row, expected, static_sig, tokens, topk, recv_cap_rows);
    else
        hipLaunchKernelGGL(moe_dispatch_signal_kernel<true>, dim3(sig_blocks, 1, (unsigned)nvshmem_n_pes()), dim3(1024),
                           0, (hipStream_t)stream, dest_pe, dest_row, expected, sig, tokens, topk, recv_cap_rows);
    return perftest::launch_status("moe_dispatch_signal");
}

int nvshmem_perftest_moe_dispatch_pieces(void *recv, size_t recv_cap_rows, const void *send,
                                         const int32_t *dest_pe, const int64_t *dest_row,
                                         const uint64_t *expected, uint64_t *sig, int tokens, int topk,
                                         size_t row_bytes, int piece_bytes, int threads, void *stream) {
    return dispatch_pieces(recv, recv_cap_rows, send, dest_pe, dest_row, expected, sig, nullptr, tokens, topk,
                           row_bytes, piece_bytes, threads, stream);
}

int nvshmem_perftest_moe_dispatch_pieces_static(void *recv, size_t recv_cap_rows, const void *send,
                                                const int32_t *dest_pe, const int64_t *dest_row,
                                                const uint64_t *expected, int tokens, int topk,
                                                size_t row_bytes, int piece_bytes, int threads,
                                                void *stream) {
    if (!perftest::ready()) return NVSHMEMX_ERROR_INVALID_VALUE;
    if (nvshmem_n_pes() > kStaticSignalPes) {
        fprintf(stderr, "nvshmem_perftest_moe_dispatch_pieces_static: %d PEs, the static signal words hold %d; "
                        "use nvshmem_perftest_moe_dispatch_pieces with signal words of your own\n",
                nvshmem_n_pes(), kStaticSignalPes);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    const int dev = current_device();
    if (dev < 0) return NVSHMEMX_ERROR_INTERNAL;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &capture) != hipSuccess) {
        (void)hipGetLastError();
        capture = hipStreamCaptureStatusNone;
    }
    uint64_t *words = scratch_address(dev, capture == hipStreamCaptureStatusNone);
    if (!words) return NVSHMEMX_ERROR_INTERNAL;
    // every call on a device uses the same words: two host threads inside the call at once are refused (calls
    // whose kernels overlap on the GPU from different streams cannot be seen from here and are the caller's
    // to avoid)
    if (scratch_calls_in_progress[dev].fetch_add(1) != 0) {
        scratch_calls_in_progress[dev].fetch_sub(1);
        fprintf(stderr, "nvshmem_perftest_moe_dispatch_pieces_static: another thread is inside this call on device %d; "
                        "the static signal words serve one call at a time\n", dev);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    const int rc = dispatch_pieces(recv, recv_cap_rows, send, dest_pe, dest_row, expected, nullptr, words, tokens, topk,
                                   row_bytes, piece_bytes, threads, stream);
    scratch_calls_in_progress[dev].fetch_sub(1);
    return rc;
}

int nvshmem_perftest_static_init(void) {
    const int dev = current_device();
    if (dev < 0) return NVSHMEMX_ERROR_INTERNAL;
    return scratch_address(dev, true) ? 0 : NVSHMEMX_ERROR_INTERNAL;
}

// piece_bytes: 0 = a work item is a whole row; 1024 / 2048 / 4096 (wavefront scope only) = a work
// item is that many bytes of a row.  With one wavefront per block and 2 KiB items every block moves
// one short piece and exits, which the memory system serves faster (measured 6.06 TB/s against
// 5.3 TB/s for whole 14 KiB rows).
int nvshmem_perftest_moe_combine_pieces(void *out, const void *recv, size_t recv_cap_rows,
                                        const int32_t *dest_pe, const int64_t *dest_row, int tokens,
                                        int topk, size_t row_bytes, int piece_bytes, int blocks_per_pe,
                                        int threads, int scope, void *stream) {
    const bool warp = scope == NVSHMEM_PERFTEST_SCOPE_WARP;
    if (!warp && scope != NVSHMEM_PERFTEST_SCOPE_BLOCK) return NVSHMEMX_ERROR_INVALID_VALUE;
    if (piece_bytes != 0 && (!warp || (piece_bytes != 1024 && piece_bytes != 2048 && piece_bytes != 4096)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if (!moe_args_ok(dest_pe, dest_row, tokens, topk, row_bytes, blocks_per_pe, threads, warp) ||
        !perftest::check_range(out, (size_t)tokens * (size_t)topk * row_bytes) ||
        !perftest::check_range(recv, recv_cap_rows * row_bytes))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if (piece_bytes > 0 &&
        (size_t)tokens * (size_t)topk * ((row_bytes + (size_t)piece_bytes - 1) / (size_t)piece_bytes) +
                (size_t)blocks_per_pe * (size_t)(threads / NVSHMEMI_WARP_SIZE) > 0xffffffffull)
        return NVSHMEMX_ERROR_INVALID_VALUE;   // the kernel counts work items in 32 bits
    const dim3 grid((unsigned)blocks_per_pe, 1, (unsigned)nvshmem_n_pes());
#define LAUNCH_COMBINE(...)                                                                        \
    hipLaunchKernelGGL((moe_combine_kernel<__VA_ARGS__>), grid, dim3(threads), 0, (hipStream_t)stream, \
                       (char *)out, (const char *)recv, dest_pe, dest_row, tokens, topk, row_bytes,    \
                       recv_cap_rows)
    if (piece_bytes == 1024) LAUNCH_COMBINE(true, 1024);
    else if (piece_bytes == 2048) LAUNCH_COMBINE(true, 2048);
    else if (piece_bytes == 4096) LAUNCH_COMBINE(true, 4096);
    else if (warp) LAUNCH_COMBINE(true, 0);
    else LAUNCH_COMBINE(false, 0);
#undef LAUNCH_COMBINE
    return perftest::launch_status("moe_combine");
}

int nvshmem_perftest_moe_combine_ex(void *out, const void *recv, size_t recv_cap_rows, const int32_t *dest_pe,
                                    const int64_t *dest_row, int tokens, int topk,
                                    size_t row_bytes, int blocks_per_pe, int threads, int scope,
                                    void *stream) {
    return nvshmem_perftest_moe_combine_pieces(out, recv, recv_cap_rows, dest_pe, dest_row, tokens, topk,
                                               row_bytes, 0, blocks_per_pe, threads, scope, stream);
}

int nvshmem_perftest_moe_combine(void *out, const void *recv, size_t recv_cap_rows, const int32_t *dest_pe,
                                 const int64_t *dest_row, int tokens, int topk, size_t row_bytes,
                                 int blocks_per_pe, int threads, void *stream) {
    return nvshmem_perftest_moe_combine_ex(out, recv, recv_cap_rows, dest_pe, dest_row, tokens, topk, row_bytes,
                                           blocks_per_pe, threads, NVSHMEM_PERFTEST_SCOPE_WARP,
                                           stream);
}

int nvshmem_perftest_moe_exchange_offsets(const int64_t *counts, int64_t *seg_base,
                                          int64_t *recv_rows, int num_experts, void *stream) {
    const int np = nvshmem_n_pes();
    if (!perftest::ready() || num_experts < np || num_experts % np ||
        (size_t)num_experts * np * sizeof(int64_t) > 64 * 1024 ||
        !perftest::check_range(counts, sizeof(int64_t) * (size_t)num_experts) ||
        !perftest::check_range(seg_base, sizeof(int64_t) * (size_t)num_experts * np) ||
        !perftest::check_range(recv_rows, sizeof(int64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    hipLaunchKernelGGL(moe_exchange_offsets_kernel, dim3(1, 1, (unsigned)np), dim3(256),
                       (size_t)num_experts * np * sizeof(int64_t), (hipStream_t)stream, counts,
                       seg_base, recv_rows, num_experts);
    return perftest::launch_status("moe_exchange_offsets");
}

}  // extern "C"
