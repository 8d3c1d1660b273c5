// Point-to-point kernels written against the public device API: ring put/get in the three scopes,
// scalar p/g, element-wise p/g/store/atomic-add bandwidth, signal operations, bounded waits, put_signal ping-pong and the ring allreduce built
// from put_signal + signal_wait_until.
//
// Counterparts in the reference tree: perftest/device/pt-to-pt/shmem_put_bw.cu:21-60,
// perftest/device/pt-to-pt/shmem_put_signal_ping_pong_latency.cu:29-49, examples/put-block.cu:30-60,
// examples/ring-reduce.cu:88-144.
#include <hip/hip_runtime.h>

#include "nvshmem_perftest.h"
#include "nvshmemx.h"
#include "perftest_common.hpp"

namespace {

// Slice [off, off+len) of a `bytes` long message owned by part `idx` of `parts`.
__device__ __forceinline__ bool slice_of(size_t bytes, size_t parts, size_t idx, size_t *off,
                                         size_t *len) {
    if (bytes < parts) {
        *off = 0;
        *len = bytes;
        return idx == 0;
    }
    const size_t per = bytes / parts;
    *off = idx * per;
    *len = (idx == parts - 1) ? bytes - *off : per;
    return true;
}

// `per_block` = bytes / gridDim.x, divided once on the host: a block that moves a few KiB should
// not spend its time in a 64-bit division.
template <int SCOPE, bool GET>
__global__ void ring_rma_kernel(char *dest, const char *src, size_t bytes, size_t per_block) {
    const int me = nvshmem_my_pe();
    const int peer = (me + 1 == nvshmem_n_pes()) ? 0 : me + 1;
    size_t off, len;
    if (per_block == 0) {  // fewer bytes than blocks: block 0 moves everything
        if (blockIdx.x != 0) return;
        off = 0;
        len = bytes;
    } else {
        off = (size_t)blockIdx.x * per_block;
        len = (blockIdx.x == gridDim.x - 1) ? bytes - off : per_block;
    }
    if (SCOPE == NVSHMEM_PERFTEST_SCOPE_BLOCK) {
        if (GET) nvshmemx_getmem_block(dest + off, src + off, len, peer);
        else nvshmemx_putmem_block(dest + off, src + off, len, peer);
    } else if (SCOPE == NVSHMEM_PERFTEST_SCOPE_WARP) {
        const size_t waves = (blockDim.x + NVSHMEMI_WARP_SIZE - 1) / NVSHMEMI_WARP_SIZE;
        // the wavefront's index as a scalar: the slice bounds and the copy's branches on them then
        // stay in scalar registers, as they do in the block scope
        const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x / NVSHMEMI_WARP_SIZE);
        size_t woff = 0, wlen = len;
        if (waves > 1 && !slice_of(len, waves, wave, &woff, &wlen)) return;
        if (GET) nvshmemx_getmem_warp(dest + off + woff, src + off + woff, wlen, peer);
        else nvshmemx_putmem_warp(dest + off + woff, src + off + woff, wlen, peer);
    } else {
        size_t toff, tlen;
        if (!slice_of(len, blockDim.x, threadIdx.x, &toff, &tlen)) return;
        if (GET) nvshmem_getmem(dest + off + toff, src + off + toff, tlen, peer);
        else nvshmem_putmem(dest + off + toff, src + off + toff, tlen, peer);
    }
}

__global__ void p_g_kernel(uint64_t *words, uint64_t *out, uint64_t value_base) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    nvshmem_uint64_p(words + me, value_base + (uint64_t)me, (me + 1) % np);
    nvshmem_barrier_all();
    uint64_t *mine = (uint64_t *)nvshmem_ptr(out, me);
    for (int q = 0; q < np; ++q) mine[q] = nvshmem_uint64_g(words + (q + np - 1) % np, q);
}

// out is plain device memory here (used as it is): [z] = the PE block z acts as, [64 + z] = nvshmem_n_pes()
__global__ void pe_identity_kernel(int *out) {
    out[blockIdx.z] = nvshmem_my_pe();
    out[64 + blockIdx.z] = nvshmem_n_pes();
}

__global__ void signal_op_kernel(uint64_t *sig, uint64_t value, int sig_op, int reps) {
    const int peer = (nvshmem_my_pe() + 1) % nvshmem_n_pes();
    for (int r = 0; r < reps; ++r) nvshmemx_signal_op(sig, value, sig_op, peer);
}

__global__ void signal_wait_kernel(uint64_t *sig, int cmp, uint64_t cmp_value, uint64_t *out) {
    const uint64_t got = nvshmem_signal_wait_until(sig, cmp, cmp_value);
    ((uint64_t *)nvshmem_ptr(out, nvshmem_my_pe()))[0] = got;
}

__global__ void pingpong_kernel(char *data, uint64_t *sig, size_t bytes, int iters) {
    const int me = nvshmem_my_pe();
    if (me > 1) return;
    for (int i = 1; i <= iters; ++i) {
        if (me == 0) {
            nvshmemx_putmem_signal_block(data, data, bytes, sig, (uint64_t)i, NVSHMEM_SIGNAL_SET, 1);
            if (threadIdx.x == 0) nvshmem_signal_wait_until(sig, NVSHMEM_CMP_EQ, (uint64_t)i);
            __syncthreads();
        } else {
            if (threadIdx.x == 0) nvshmem_signal_wait_until(sig, NVSHMEM_CMP_EQ, (uint64_t)i);
            __syncthreads();
            nvshmemx_putmem_signal_block(data, data, bytes, sig, (uint64_t)i, NVSHMEM_SIGNAL_SET, 0);
        }
    }
}

// Ordering check for put-with-signal: even PEs stream `iters` messages to their odd neighbours
// through a ring of `slots` buffers per block.  Message i of block b holds words mix(i, b, j); the
// receiver waits for the i-th signal, reads the slot at once and counts the words that differ, then
// returns a credit.  A signal that overtook its payload shows up as a word of an older message.
__device__ __forceinline__ uint64_t stream_word(uint64_t i, uint64_t b, uint64_t j) {
    uint64_t x = (i + 1) * 0x9E3779B97F4A7C15ull ^ (b + 1) * 0xC2B2AE3D27D4EB4Full ^ j * 0x165667B19E3779F9ull;
    x ^= x >> 29;
    return x * 0xBF58476D1CE4E5B9ull;
}
template <int SCOPE>
__global__ void put_signal_stream_kernel(char *data, char *stage, uint64_t *sig, uint64_t *errors,
                                         size_t bytes, int slots, int iters, int sig_op) {
    const int me = nvshmem_my_pe(), peer = me ^ 1;
    if (peer >= nvshmem_n_pes()) return;
    const bool sender = (me & 1) == 0;
    const size_t b = blockIdx.x, words = bytes / 8;
    char *slot_base = data + b * (size_t)slots * bytes;
    char *my_stage = stage + b * bytes;
    uint64_t *data_sig = sig + 2 * b, *credit = sig + 2 * b + 1;
    unsigned long long bad = 0;
    for (int i = 0; i < iters; ++i) {
        char *slot = slot_base + (size_t)(i % slots) * bytes;
        if (sender) {
            if (i >= slots) {
                if (threadIdx.x == 0) nvshmem_signal_wait_until(credit, NVSHMEM_CMP_GE, (uint64_t)(i - slots + 1));
                __syncthreads();
            }
            uint64_t *st = (uint64_t *)nvshmem_ptr(my_stage, me);
            for (size_t j = threadIdx.x; j < words; j += blockDim.x) st[j] = stream_word(i, b, j);
            __syncthreads();
            if (SCOPE == NVSHMEM_PERFTEST_SCOPE_BLOCK)
                nvshmemx_putmem_signal_nbi_block(slot, my_stage, bytes, data_sig, 1, sig_op, peer);
            else if (SCOPE == NVSHMEM_PERFTEST_SCOPE_WARP)
                nvshmemx_putmem_signal_nbi_warp(slot, my_stage, bytes, data_sig, 1, sig_op, peer);
            else
                nvshmem_putmem_signal_nbi(slot, my_stage, bytes, data_sig, 1, sig_op, peer);
        } else {
            if (threadIdx.x == 0) nvshmem_signal_wait_until(data_sig, NVSHMEM_CMP_GE, (uint64_t)(i + 1));
            __syncthreads();
            const uint64_t *got = (const uint64_t *)nvshmem_ptr(slot, me);
            for (size_t j = threadIdx.x; j < words; j += blockDim.x) bad += got[j] != stream_word(i, b, j);
            __syncthreads();
            if (threadIdx.x == 0) nvshmemx_signal_op(credit, 1, NVSHMEM_SIGNAL_ADD, peer);
        }
    }
    if (bad) atomicAdd((unsigned long long *)nvshmem_ptr(errors, me), bad);
}

// every PE's copy of `words` := value, in one launch (stream ordered, unlike a memset per PE)
__global__ void fill_words_kernel(uint64_t *words, uint64_t value, size_t n) {
    uint64_t *mine = (uint64_t *)nvshmem_ptr(words, nvshmem_my_pe());
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        mine[i] = value;
}

// Point-to-point latency loops in the shape of the reference's perftest/device/pt-to-pt programs:
// PE 0 acts on PE 1 `iters` times (kinds 0-4: shmem_put_latency.cu, shmem_get_latency.cu,
// shmem_p_latency.cu, shmem_g_latency.cu, shmem_atomic_latency.cu), or PE 0 and PE 1 bounce a word
// (kinds 5-7: shmem_signal_ping_pong_latency.cu, shmem_p_ping_pong_latency.cu,
// shmem_atomic_ping_pong_latency.cu).  sig holds two words per PE.
__global__ void pt2pt_latency_kernel(int what, char *data, uint64_t *sig, size_t bytes, int iters) {
    const int me = nvshmem_my_pe();
    if (me > 1) return;
    const int peer = 1 - me;
    if (what <= NVSHMEM_PERFTEST_LAT_ATOMIC) {
        if (me != 0) return;
        uint64_t acc = 0;
        for (int i = 1; i <= iters; ++i) {
            switch (what) {
                case NVSHMEM_PERFTEST_LAT_PUT:
                    nvshmemx_putmem_block(data, data, bytes, peer);
                    nvshmem_quiet();
                    break;
                case NVSHMEM_PERFTEST_LAT_GET:
                    nvshmemx_getmem_block(data, data, bytes, peer);
                    break;
                case NVSHMEM_PERFTEST_LAT_P:
                    if (threadIdx.x == 0) {
                        nvshmem_uint64_p(sig, (uint64_t)i, peer);
                        nvshmem_quiet();
                    }
                    break;
                case NVSHMEM_PERFTEST_LAT_G:
                    if (threadIdx.x == 0) acc += nvshmem_uint64_g(sig, peer);
                    break;
                default:
                    // every fetch depends on the one before: a chain of round trips
                    if (threadIdx.x == 0) acc = nvshmem_uint64_atomic_fetch_add(sig, 1 + (acc >> 63), peer);
                    break;
            }
        }
        if (threadIdx.x == 0 && what >= NVSHMEM_PERFTEST_LAT_G) ((uint64_t *)nvshmem_ptr(sig, me))[1] = acc;
        return;
    }
    if (threadIdx.x != 0) return;
    for (int i = 1; i <= iters; ++i) {
        if (me == 1) nvshmem_uint64_wait_until(sig, NVSHMEM_CMP_EQ, (uint64_t)i);
        switch (what) {
            case NVSHMEM_PERFTEST_LAT_SIGNAL_PINGPONG:
                nvshmemx_signal_op(sig, (uint64_t)i, NVSHMEM_SIGNAL_SET, peer);
                break;
            case NVSHMEM_PERFTEST_LAT_P_PINGPONG:
                nvshmem_uint64_p(sig, (uint64_t)i, peer);
                break;
            default:
                nvshmem_uint64_atomic_inc(sig, peer);
                break;
        }
        if (me == 0) nvshmem_uint64_wait_until(sig, NVSHMEM_CMP_EQ, (uint64_t)i);
    }
}

// Ring allreduce: the partial sum travels PE 0 -> 1 -> ... -> n-1 chunk by chunk (reduce phase),
// then the finished chunks travel n-1 -> 0 -> ... -> n-2 (broadcast phase).  A signal word per
// block counts the chunks that have arrived.
__global__ void ring_reduce_kernel(int32_t *dst, const int32_t *src, size_t nreduce,
                                   uint64_t *signal, size_t chunk_elems) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    const int peer = (me + 1) % np;
    const size_t per_block = nreduce / gridDim.x;
    const size_t chunks = per_block / chunk_elems;
    dst += (size_t)blockIdx.x * per_block;
    src += (size_t)blockIdx.x * per_block;
    signal += blockIdx.x;
    int32_t *my_dst = (int32_t *)nvshmem_ptr(dst, me);
    const int32_t *my_src = (const int32_t *)nvshmem_ptr(src, me);

    for (size_t c = 0; c < chunks; ++c) {
        const size_t at = c * chunk_elems;
        if (me != 0) {
            if (threadIdx.x == 0) nvshmem_signal_wait_until(signal, NVSHMEM_CMP_GE, c + 1);
            __syncthreads();
            for (size_t i = threadIdx.x; i < chunk_elems; i += blockDim.x)
                my_dst[at + i] = (int32_t)((uint32_t)my_dst[at + i] + (uint32_t)my_src[at + i]);
            __syncthreads();
        }
        nvshmemx_int32_put_signal_nbi_block(dst + at, (me == 0) ? src + at : dst + at, chunk_elems,
                                            signal, 1, NVSHMEM_SIGNAL_ADD, peer);
    }
    for (size_t c = 0; c < chunks; ++c) {
        const size_t at = c * chunk_elems;
        if (me < np - 1) {
            if (threadIdx.x == 0)
                nvshmem_signal_wait_until(signal, NVSHMEM_CMP_GE, (me == 0) ? c + 1 : chunks + c + 1);
            __syncthreads();
        }
        if (me < np - 2)
            nvshmemx_int32_put_signal_nbi_block(dst + at, dst + at, chunk_elems, signal, 1,
                                                NVSHMEM_SIGNAL_ADD, peer);
    }
    __syncthreads();
    if (threadIdx.x == 0) *(uint64_t *)nvshmem_ptr(signal, me) = 0;  // ready for the next run
}

// One-sided stream probes for hardware counters: the deep rounds of a long block-scoped copy with one side
// removed.  Every block reads (WRITE false) or writes (WRITE true) its contiguous slice of the calling
// PE's buffer, 8 vectors per lane and round, wavefront w the w-th KiB of every 16 KiB.  What they show is
// how many requests a compute unit keeps in flight when loads and stores do not share its queues.
template <int WRITE>   // 0 read, 1 write with streaming (nt) stores, 2 write with write-through (sc1 nt) stores
__global__ __launch_bounds__(1024) void stream_probe_kernel(char *buf, size_t bytes, size_t per_block) {
    char *mine = (char *)nvshmem_ptr(buf, nvshmem_my_pe()) + (size_t)blockIdx.x * per_block;
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane_off = (threadIdx.x & 63u) * 16u;
    const size_t step = (size_t)blockDim.x * 16, per_round = 8 * step;
    nvshmemi_v4u acc = {0u, 0u, 0u, 0u};
    for (size_t r = 0; r + per_round <= per_block; r += per_round) {
        char *p = mine + r + (size_t)wave * 1024 + lane_off;
        if (WRITE) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const nvshmemi_v4u v = {(unsigned)r, threadIdx.x, (unsigned)u, blockIdx.x};
                if (WRITE == 2) nvshmemi_amd_stream_store16<NVSHMEMI_AMD_STORE_WRITE_THROUGH>(p + u * step, v);
                else __builtin_nontemporal_store(v, reinterpret_cast<nvshmemi_v4u *>(p + u * step));
            }
        } else {
            nvshmemi_v4u v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(reinterpret_cast<const nvshmemi_v4u *>(p + u * step));
#pragma unroll
            for (int u = 0; u < 8; ++u) acc ^= v[u];
        }
    }
    // (keeps the loads alive; random data never matches)
    if (!WRITE && acc.x == 0x9E3779B1u && acc.y == 0x85EBCA77u && acc.z == 0xC2B2AE3Du && acc.w == 1u)
        *reinterpret_cast<nvshmemi_v4u *>(mine) = acc;
}

// Boundary between workloads in a profiler trace: does nothing, has a name of its own.
__global__ void profile_marker_kernel() {}

// Calibration kernel for hardware counters: a plain copy of a known size that uses nothing of the
// NVSHMEM API (one 16-byte vector per thread).
__global__ void plain_copy_kernel(nvshmemi_v4u *dst, const nvshmemi_v4u *src, size_t nvec) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < nvec) dst[i] = src[i];
}

// Element-wise bandwidth in the shape of the reference's shmem_p_bw.cu:43-84, shmem_g_bw.cu,
// shmem_st_bw.cu and shmem_atomic_bw.cu: every thread moves single elements, consecutive threads
// consecutive elements, every PE to (P, ST, ADD) or from (G) its right neighbour.
template <typename T> struct element_api;
#define ELEMENT_API(T, NAME)                                                                          \
    template <> struct element_api<T> {                                                               \
        static __device__ __forceinline__ void p(T *d, T v, int pe) { nvshmem_##NAME##_p(d, v, pe); } \
        static __device__ __forceinline__ T g(const T *s, int pe) { return nvshmem_##NAME##_g(s, pe); } \
    };
ELEMENT_API(uint8_t, uint8)
ELEMENT_API(uint16_t, uint16)
ELEMENT_API(uint32_t, uint32)
ELEMENT_API(uint64_t, uint64)
#undef ELEMENT_API
__device__ __forceinline__ void element_add(uint8_t *, uint8_t, int) {}
__device__ __forceinline__ void element_add(uint16_t *, uint16_t, int) {}
__device__ __forceinline__ void element_add(uint32_t *d, uint32_t v, int pe) { nvshmem_uint32_atomic_add(d, v, pe); }
__device__ __forceinline__ void element_add(uint64_t *d, uint64_t v, int pe) { nvshmem_uint64_atomic_add(d, v, pe); }

template <typename T, int WHAT>
__global__ void element_bw_kernel(T *dest, const T *src, size_t n) {
    const int me = nvshmem_my_pe();
    const int peer = (me + 1 == nvshmem_n_pes()) ? 0 : me + 1;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const T *my_src = (const T *)nvshmem_ptr(src, me);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        if (WHAT == NVSHMEM_PERFTEST_ELEMENT_P) element_api<T>::p(dest + i, my_src[i], peer);
        else if (WHAT == NVSHMEM_PERFTEST_ELEMENT_G) ((T *)nvshmem_ptr(dest, me))[i] = element_api<T>::g(src + i, peer);
        else if (WHAT == NVSHMEM_PERFTEST_ELEMENT_ST) ((T *)nvshmem_ptr(dest, peer))[i] = my_src[i];
        else element_add(dest + i, my_src[i], peer);
    }
}

template <typename T>
int launch_element(int what, void *dest, const void *src, size_t n, int blocks, int threads, hipStream_t stream) {
    const dim3 grid((unsigned)blocks, 1, (unsigned)nvshmem_n_pes());
    switch (what) {
        case NVSHMEM_PERFTEST_ELEMENT_P:
            hipLaunchKernelGGL((element_bw_kernel<T, NVSHMEM_PERFTEST_ELEMENT_P>), grid, dim3(threads), 0, stream, (T *)dest, (const T *)src, n);
            break;
        case NVSHMEM_PERFTEST_ELEMENT_G:
            hipLaunchKernelGGL((element_bw_kernel<T, NVSHMEM_PERFTEST_ELEMENT_G>), grid, dim3(threads), 0, stream, (T *)dest, (const T *)src, n);
            break;
        case NVSHMEM_PERFTEST_ELEMENT_ST:
            hipLaunchKernelGGL((element_bw_kernel<T, NVSHMEM_PERFTEST_ELEMENT_ST>), grid, dim3(threads), 0, stream, (T *)dest, (const T *)src, n);
            break;
        default:
            hipLaunchKernelGGL((element_bw_kernel<T, NVSHMEM_PERFTEST_ELEMENT_ADD>), grid, dim3(threads), 0, stream, (T *)dest, (const T *)src, n);
            break;
    }
    return perftest::launch_status("element_bw");
}

template <int SCOPE>
int launch_ring(bool is_get, char *dest, const char *src, size_t bytes, int blocks, int threads,
                hipStream_t stream) {
    const dim3 grid((unsigned)blocks, 1, (unsigned)nvshmem_n_pes());
    const size_t per_block = bytes / (size_t)blocks;
    if (is_get)
        hipLaunchKernelGGL((ring_rma_kernel<SCOPE, true>), grid, dim3(threads), 0, stream, dest, src, bytes,
                           per_block);
    else
        hipLaunchKernelGGL((ring_rma_kernel<SCOPE, false>), grid, dim3(threads), 0, stream, dest, src, bytes,
                           per_block);
    return perftest::launch_status("ring_rma");
}

}  // namespace

extern "C" {

int nvshmem_perftest_ring_rma(void *dest, const void *src, size_t bytes, int blocks_per_pe,
                              int threads, int scope, int is_get, int iters, void *stream) {
    if (!perftest::ready() || !perftest::check_launch(blocks_per_pe, threads) ||
        !perftest::check_range(dest, bytes) || !perftest::check_range(src, bytes))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if (bytes == 0) return 0;
    int rc = 0;
    for (int i = 0; i < iters && rc == 0; ++i) {
        switch (scope) {
            case NVSHMEM_PERFTEST_SCOPE_BLOCK:
                rc = launch_ring<NVSHMEM_PERFTEST_SCOPE_BLOCK>(is_get, (char *)dest, (const char *)src,
                                                               bytes, blocks_per_pe, threads,
                                                               (hipStream_t)stream);
                break;
            case NVSHMEM_PERFTEST_SCOPE_WARP:
                rc = launch_ring<NVSHMEM_PERFTEST_SCOPE_WARP>(is_get, (char *)dest, (const char *)src,
                                                              bytes, blocks_per_pe, threads,
                                                              (hipStream_t)stream);
                break;
            case NVSHMEM_PERFTEST_SCOPE_THREAD:
                rc = launch_ring<NVSHMEM_PERFTEST_SCOPE_THREAD>(is_get, (char *)dest, (const char *)src,
                                                                bytes, blocks_per_pe, threads,
                                                                (hipStream_t)stream);
                break;
            default:
                return NVSHMEMX_ERROR_INVALID_VALUE;
        }
    }
    return rc;
}

int nvshmem_perftest_element_bw(int what, int elem_bytes, void *dest, const void *src, size_t nelems,
                                int blocks_per_pe, int threads, void *stream) {
    const bool size_ok = elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8;
    if (!perftest::ready() || what < 0 || what > NVSHMEM_PERFTEST_ELEMENT_ADD || !size_ok ||
        (what == NVSHMEM_PERFTEST_ELEMENT_ADD && elem_bytes < 4) ||
        ((uintptr_t)dest % elem_bytes) || ((uintptr_t)src % elem_bytes) ||
        !perftest::check_launch(blocks_per_pe, threads) ||
        !perftest::check_range(dest, nelems * elem_bytes) || !perftest::check_range(src, nelems * elem_bytes))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if (nelems == 0) return 0;
    switch (elem_bytes) {
        case 1: return launch_element<uint8_t>(what, dest, src, nelems, blocks_per_pe, threads, (hipStream_t)stream);
        case 2: return launch_element<uint16_t>(what, dest, src, nelems, blocks_per_pe, threads, (hipStream_t)stream);
        case 4: return launch_element<uint32_t>(what, dest, src, nelems, blocks_per_pe, threads, (hipStream_t)stream);
        default: return launch_element<uint64_t>(what, dest, src, nelems, blocks_per_pe, threads, (hipStream_t)stream);
    }
}

int nvshmem_perftest_plain_copy(void *dst, const void *src, size_t bytes, void *stream) {
    if (!perftest::ready() || (bytes % 16) || ((uintptr_t)dst % 16) || ((uintptr_t)src % 16) ||
        !perftest::check_range(dst, bytes) || !perftest::check_range(src, bytes))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    const size_t nvec = bytes / 16;
    if (nvec == 0) return 0;
    hipLaunchKernelGGL(plain_copy_kernel, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (nvshmemi_v4u *)dst, (const nvshmemi_v4u *)src, nvec);
    return perftest::launch_status("plain_copy");
}

int nvshmem_perftest_stream_probe(void *buf, size_t bytes, int blocks_per_pe, int threads, int write, void *stream) {
    if (!perftest::ready() || !perftest::check_launch(blocks_per_pe, threads) || (threads % 64) || !perftest::check_range(buf, bytes) ||
        ((uintptr_t)buf % 16))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    const size_t round = (size_t)threads * 16 * 8;
    const size_t per_block = bytes / (size_t)blocks_per_pe / round * round;  // whole rounds only
    if (per_block == 0) return NVSHMEMX_ERROR_INVALID_VALUE;
    const dim3 grid((unsigned)blocks_per_pe, 1, (unsigned)nvshmem_n_pes());
    if (write == 2) hipLaunchKernelGGL(stream_probe_kernel<2>, grid, dim3(threads), 0, (hipStream_t)stream, (char *)buf, bytes, per_block);
    else if (write) hipLaunchKernelGGL(stream_probe_kernel<1>, grid, dim3(threads), 0, (hipStream_t)stream, (char *)buf, bytes, per_block);
    else hipLaunchKernelGGL(stream_probe_kernel<0>, grid, dim3(threads), 0, (hipStream_t)stream, (char *)buf, bytes, per_block);
    return perftest::launch_status("stream_probe");
}

int nvshmem_perftest_profile_marker(void *stream) {
    hipLaunchKernelGGL(profile_marker_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream);
    return perftest::launch_status("profile_marker");
}

int nvshmem_perftest_p_g(uint64_t *words, uint64_t *out, uint64_t value_base, void *stream) {
    const size_t row = sizeof(uint64_t) * (size_t)nvshmem_n_pes();
    if (!perftest::ready() || !perftest::check_range(words, row) || !perftest::check_range(out, row))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    void *args[] = {&words, &out, &value_base};
    return nvshmemx_collective_launch((const void *)p_g_kernel, dim3(1), dim3(1), args, 0,
                                      (hipStream_t)stream);
}

int nvshmem_perftest_pe_identity(int *out, int grid_z, void *stream) {
    if (!perftest::ready() || !out || grid_z < 1 || grid_z > 64) return NVSHMEMX_ERROR_INVALID_VALUE;
    hipLaunchKernelGGL(pe_identity_kernel, dim3(1, 1, (unsigned)grid_z), dim3(1), 0, (hipStream_t)stream, out);
    return perftest::launch_status("pe_identity");
}

int nvshmem_perftest_signal_op(uint64_t *sig, uint64_t value, int sig_op, int threads, int reps,
                               void *stream) {
    if (!perftest::ready() || !perftest::check_launch(1, threads) ||
        !perftest::check_range(sig, sizeof(uint64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if (sig_op != NVSHMEM_SIGNAL_SET && sig_op != NVSHMEM_SIGNAL_ADD)
        return NVSHMEMX_ERROR_INVALID_VALUE;
    hipLaunchKernelGGL(signal_op_kernel, dim3(1, 1, (unsigned)nvshmem_n_pes()), dim3(threads), 0,
                       (hipStream_t)stream, sig, value, sig_op, reps);
    return perftest::launch_status("signal_op");
}

int nvshmem_perftest_signal_wait(uint64_t *sig, int cmp, uint64_t cmp_value, uint64_t *out,
                                 void *stream) {
    if (!perftest::ready() || !perftest::check_range(sig, sizeof(uint64_t)) ||
        !perftest::check_range(out, sizeof(uint64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    hipLaunchKernelGGL(signal_wait_kernel, dim3(1, 1, (unsigned)nvshmem_n_pes()), dim3(1), 0,
                       (hipStream_t)stream, sig, cmp, cmp_value, out);
    return perftest::launch_status("signal_wait");
}

int nvshmem_perftest_put_signal_pingpong(void *data, uint64_t *sig, size_t bytes, int iters,
                                         int threads, void *stream) {
    if (!perftest::ready() || nvshmem_n_pes() < 2 || !perftest::check_launch(1, threads) ||
        !perftest::check_range(data, bytes) || !perftest::check_range(sig, sizeof(uint64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    char *d = (char *)data;
    void *args[] = {&d, &sig, &bytes, &iters};
    return nvshmemx_collective_launch((const void *)pingpong_kernel, dim3(1), dim3(threads), args,
                                      0, (hipStream_t)stream);
}

int nvshmem_perftest_put_signal_stream(void *data, void *stage, uint64_t *sig, uint64_t *errors,
                                       size_t bytes, int slots, int iters, int blocks, int scope,
                                       int sig_op, void *stream) {
    const int threads = scope == NVSHMEM_PERFTEST_SCOPE_BLOCK ? 256 : scope == NVSHMEM_PERFTEST_SCOPE_WARP ? 64 : 1;
    if (!perftest::ready() || nvshmem_n_pes() < 2 || bytes == 0 || bytes % 8 || slots < 1 || iters < 1 ||
        scope < NVSHMEM_PERFTEST_SCOPE_THREAD || scope > NVSHMEM_PERFTEST_SCOPE_BLOCK ||
        !perftest::check_launch(blocks, threads) ||
        !perftest::check_range(data, (size_t)blocks * (size_t)slots * bytes) ||
        !perftest::check_range(stage, (size_t)blocks * bytes) ||
        !perftest::check_range(sig, 2 * sizeof(uint64_t) * (size_t)blocks) ||
        !perftest::check_range(errors, sizeof(uint64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    const int op = sig_op & NVSHMEMI_AMD_SIGNAL_OP_MASK;
    if (op != NVSHMEM_SIGNAL_ADD) return NVSHMEMX_ERROR_INVALID_VALUE;
    char *d = (char *)data, *st = (char *)stage;
    void *args[] = {&d, &st, &sig, &errors, &bytes, &slots, &iters, &sig_op};
    const void *fn = scope == NVSHMEM_PERFTEST_SCOPE_BLOCK  ? (const void *)put_signal_stream_kernel<NVSHMEM_PERFTEST_SCOPE_BLOCK>
                     : scope == NVSHMEM_PERFTEST_SCOPE_WARP ? (const void *)put_signal_stream_kernel<NVSHMEM_PERFTEST_SCOPE_WARP>
                                                            : (const void *)put_signal_stream_kernel<NVSHMEM_PERFTEST_SCOPE_THREAD>;
    return nvshmemx_collective_launch(fn, dim3(blocks), dim3(threads), args, 0, (hipStream_t)stream);
}

int nvshmem_perftest_fill_words(uint64_t *words, uint64_t value, size_t nwords, void *stream) {
    if (!perftest::ready() || !perftest::check_range(words, nwords * sizeof(uint64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if (nwords == 0) return 0;
    const unsigned blocks = (unsigned)((nwords + 255) / 256 < 1024 ? (nwords + 255) / 256 : 1024);
    hipLaunchKernelGGL(fill_words_kernel, dim3(blocks, 1, (unsigned)nvshmem_n_pes()), dim3(256), 0,
                       (hipStream_t)stream, words, value, nwords);
    return perftest::launch_status("fill_words");
}

int nvshmem_perftest_pt2pt_latency(int what, void *data, uint64_t *sig, size_t bytes, int iters,
                                   int threads, void *stream) {
    if (!perftest::ready() || nvshmem_n_pes() < 2 || what < 0 || what > NVSHMEM_PERFTEST_LAT_ATOMIC_PINGPONG ||
        iters < 1 || !perftest::check_launch(1, threads) || !perftest::check_range(data, bytes) ||
        !perftest::check_range(sig, 2 * sizeof(uint64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    char *d = (char *)data;
    void *args[] = {&what, &d, &sig, &bytes, &iters};
    return nvshmemx_collective_launch((const void *)pt2pt_latency_kernel, dim3(1), dim3(threads), args,
                                      0, (hipStream_t)stream);
}

int nvshmem_perftest_ring_reduce(int32_t *dst, const int32_t *src, size_t nreduce,
                                 uint64_t *signal, size_t chunk_elems, int blocks, int threads,
                                 void *stream) {
    if (!perftest::ready() || !perftest::check_launch(blocks, threads) || chunk_elems == 0 ||
        nreduce % ((size_t)blocks * chunk_elems) != 0 ||
        !perftest::check_range(dst, nreduce * sizeof(int32_t)) ||
        !perftest::check_range(src, nreduce * sizeof(int32_t)) ||
        !perftest::check_range(signal, sizeof(uint64_t) * (size_t)blocks))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    void *args[] = {&dst, &src, &nreduce, &signal, &chunk_elems};
    return nvshmemx_collective_launch((const void *)ring_reduce_kernel, dim3(blocks), dim3(threads),
                                      args, 0, (hipStream_t)stream);
}

}  // extern "C"
