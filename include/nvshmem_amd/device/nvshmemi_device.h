/*
 * Device-side building blocks of the data-movement path for gfx950 (wavefront64).
 * Header-only: everything is inlined into the caller's kernel, as in the reference, whose device
 * layer is src/include/non_abi/device/{common,threadgroup,wait,coll}.
 *
 * Logical PEs.  A kernel started through nvshmemx_collective_launch has gridDim.z == npes and a
 * block acts as PE blockIdx.z.  Symmetric pointers in kernel arguments are canonical (PE 0 slice)
 * addresses; API calls translate them: a remote operand goes to PE `pe`'s slice, a local operand
 * that lies in slice 0 goes to the calling PE's slice, any other address is used as it is.
 * Code that dereferences a symmetric pointer itself localises it with nvshmem_ptr(p, nvshmem_my_pe()).
 */
#ifndef NVSHMEM_AMD_DEVICE_INTERNAL_H
#define NVSHMEM_AMD_DEVICE_INTERNAL_H

#if !defined(__HIPCC__)
#error "the NVSHMEM device API needs hipcc"
#endif

#include <hip/hip_runtime.h>
#include <type_traits>
#include "../nvshmem_host_api.h"
#include "../nvshmem_types.h"

/* One private copy per translation unit.  The unit registers a callback that copies the host
 * library's state block into its copy; the library calls every registered callback whenever the
 * state changes. */
static __constant__ nvshmemi_device_state_t nvshmemi_device_state_d;

namespace nvshmemi_amd {
static int push_state(const nvshmemi_device_state_t *host_copy) {
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(nvshmemi_device_state_d), host_copy,
                                  sizeof(nvshmemi_device_state_t), 0, hipMemcpyHostToDevice);
}
struct state_registrar {
    state_registrar() { nvshmemi_amd_register_state_updater(&push_state); }
    ~state_registrar() { nvshmemi_amd_unregister_state_updater(&push_state); }
};
static state_registrar state_registrar_instance;
}  // namespace nvshmemi_amd

#define NVSHMEMI_DEVICE_INLINE __device__ __forceinline__

/* ------------------------------------------------------------------------------------------------
 * Thread groups (reference threadgroup/nvshmemi_common_device_defines.cuh:32-120)
 * ---------------------------------------------------------------------------------------------- */
enum nvshmemi_threadgroup_t {
    NVSHMEMI_THREADGROUP_THREAD = 0,
    NVSHMEMI_THREADGROUP_WARP = 1,
    NVSHMEMI_THREADGROUP_BLOCK = 2
};

// Work-group extents through the compiler builtins: three scalar loads at the top of the kernel.
// (blockDim.z goes through a select between the full and the remainder group size, a vector load
// that every block waits on before its first copy instruction.)
NVSHMEMI_DEVICE_INLINE unsigned nvshmemi_amd_block_size() {
    return (unsigned)__builtin_amdgcn_workgroup_size_x() * __builtin_amdgcn_workgroup_size_y() *
           __builtin_amdgcn_workgroup_size_z();
}
NVSHMEMI_DEVICE_INLINE unsigned nvshmemi_amd_block_tid() {
    return threadIdx.x + (unsigned)__builtin_amdgcn_workgroup_size_x() *
                             (threadIdx.y + (unsigned)__builtin_amdgcn_workgroup_size_y() * threadIdx.z);
}

// A wavefront holds 64 consecutive threads of the block's linear order, so a thread's index in its
// wavefront is its lane number and the wavefront's size is the number of lanes it was started with
// (fewer than 64 only in the last wavefront of a block whose size is no multiple of 64).  Neither
// needs the block's extents, which cost a wavefront that moves 1 KiB a measurable wait (a put of
// 1 KiB per wavefront: 385 GB/s per PE with the extents, 430 without).  Warp-scoped calls are made by
// all lanes of the wavefront, so the lanes active at the call are the lanes it was started with.
NVSHMEMI_DEVICE_INLINE unsigned nvshmemi_amd_lane_id() {
    return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}
NVSHMEMI_DEVICE_INLINE unsigned nvshmemi_amd_lanes_in_wavefront() {
    return (unsigned)__builtin_popcountll(__builtin_amdgcn_ballot_w64(true));
}

template <int SCOPE>
NVSHMEMI_DEVICE_INLINE int nvshmemi_thread_id_in_threadgroup() {
    if (SCOPE == NVSHMEMI_THREADGROUP_WARP) return (int)nvshmemi_amd_lane_id();
    if (SCOPE == NVSHMEMI_THREADGROUP_BLOCK) return (int)nvshmemi_amd_block_tid();
    return 0;
}

template <int SCOPE>
NVSHMEMI_DEVICE_INLINE int nvshmemi_threadgroup_size() {
    if (SCOPE == NVSHMEMI_THREADGROUP_WARP) return (int)nvshmemi_amd_lanes_in_wavefront();
    if (SCOPE == NVSHMEMI_THREADGROUP_BLOCK) return (int)nvshmemi_amd_block_size();
    return 1;
}

template <int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_threadgroup_sync() {
    if (SCOPE == NVSHMEMI_THREADGROUP_WARP) {
        /* A wavefront runs in lock step; this only orders its memory operations. */
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    } else if (SCOPE == NVSHMEMI_THREADGROUP_BLOCK) {
        __syncthreads();
    }
}

/* Wait until this wavefront's outstanding vector memory operations have completed
 * (s_waitcnt vmcnt(0), gfx9 encoding: lgkmcnt and expcnt left at their maxima). */
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_wait_vm() { __builtin_amdgcn_s_waitcnt(0x0F70); }

/* ------------------------------------------------------------------------------------------------
 * PE identity and address translation
 * (reference nvshmemi_ptr, common/nvshmemi_common_device.cuh:578-590, and the inline
 * `peer_base + (ptr - heap_base)` of every RMA call, e.g. :493-498)
 * ---------------------------------------------------------------------------------------------- */
NVSHMEMI_DEVICE_INLINE int nvshmemi_amd_my_pe() {
    return (gridDim.z == (unsigned)nvshmemi_device_state_d.npes) ? (int)blockIdx.z
                                                                 : nvshmemi_device_state_d.mype;
}
NVSHMEMI_DEVICE_INLINE int nvshmemi_amd_n_pes() { return nvshmemi_device_state_d.npes; }

/* Offset inside its slice of an address anywhere in the heap (canonical addresses, PE 0's slice, are
 * their own offset).  The slice index floor(d / size) is computed without a division or a branch: size
 * is a multiple of 2 MiB, so it equals floor((d >> 21) / (size >> 21)), and for the fewer than 2^18
 * units of a heap of at most 512 GiB that quotient is ((d >> 21) * heap_magic) >> 40 with
 * heap_magic = floor(2^40 / (size >> 21)) + 1 (the error of the reciprocal, below 2^-22, is smaller than
 * the 1 / (size >> 21) that separates a quotient from the next integer).  A dozen scalar instructions
 * when the address is wave-uniform; a compare-and-divide form cost the small collectives 0.1-0.2 us. */
NVSHMEMI_DEVICE_INLINE uint64_t nvshmemi_amd_slice_offset(const void *sym) {
    const uint64_t d = (uint64_t)((const char *)sym - nvshmemi_device_state_d.heap_base);
    const uint32_t slice =
        (uint32_t)(((uint64_t)(uint32_t)(d >> 21) * nvshmemi_device_state_d.heap_magic) >> 40);
    return d - (uint64_t)slice * nvshmemi_device_state_d.heap_size;
}
/* Address of PE `pe`'s copy of the symmetric object at `sym` (an address in any PE's slice). */
NVSHMEMI_DEVICE_INLINE char *nvshmemi_amd_remote(const void *sym, int pe) {
    return nvshmemi_device_state_d.heap_base + (uint64_t)(unsigned)pe * nvshmemi_device_state_d.heap_size +
           nvshmemi_amd_slice_offset(sym);
}

/* Local operand: a canonical address means "my copy"; anything else is taken literally. */
NVSHMEMI_DEVICE_INLINE char *nvshmemi_amd_local(const void *p) {
    const uint64_t off = (uint64_t)((const char *)p - nvshmemi_device_state_d.heap_base);
    if (off < nvshmemi_device_state_d.heap_size)
        return nvshmemi_device_state_d.heap_base +
               (uint64_t)(unsigned)nvshmemi_amd_my_pe() * nvshmemi_device_state_d.heap_size + off;
    return (char *)p;
}

NVSHMEMI_DEVICE_INLINE void *nvshmemi_ptr(const void *ptr, int pe) {
    const uint64_t off = (uint64_t)((const char *)ptr - nvshmemi_device_state_d.heap_base);
    if (pe >= 0 && pe < nvshmemi_device_state_d.npes &&
        off < (uint64_t)(unsigned)nvshmemi_device_state_d.npes * nvshmemi_device_state_d.heap_size)
        return nvshmemi_amd_remote(ptr, pe);
    return nullptr;
}

/* ------------------------------------------------------------------------------------------------
 * Copy engine (reference nvshmemi_memcpy_threadgroup, common/nvshmemi_common_device.cuh:254-349)
 *
 * Byte-exact copy by the lanes of one thread group.  Where the reference picks the widest element
 * both pointers are aligned to and cascades, this version always stores 16-byte vectors: a byte
 * head brings dst to a 16-byte boundary, the body issues four (long copies: sixteen) independent
 * dwordx4 loads per lane before the first store (gfx950 accepts unaligned vector loads, so a src that
 * is not co-aligned only costs extra cache-line touches, not narrower instructions), and a byte tail
 * finishes.
 * ---------------------------------------------------------------------------------------------- */
typedef unsigned int nvshmemi_v4u __attribute__((ext_vector_type(4)));
typedef nvshmemi_v4u __attribute__((aligned(1))) nvshmemi_v4u_unaligned;

/* Vectors per lane and round of the ordinary body.  A translation unit whose calls move rows of a known
 * size does best with the number of vectors a lane moves per call - a 14 KiB row per wavefront: 14 - so
 * that a call is one run of loads followed by one run of stores (the token dispatch with a signal per row:
 * 4.53 TB/s at 8, 4.90 at 14; the price is 4 vector registers per vector). */
#ifndef NVSHMEMI_AMD_COPY_UNROLL
#define NVSHMEMI_AMD_COPY_UNROLL 4
#endif
/* Long copies - a lane owns at least NVSHMEMI_AMD_COPY_DEEP_MIN vectors - run rounds of
 * NVSHMEMI_AMD_COPY_DEEP_UNROLL vectors per lane first (0 switches them off).  Eight is what fits the
 * registers the rest of the engine needs anyway.  Sixteen takes 30 more vector registers (82 in all: five
 * wavefronts per SIMD instead of eight), which cost kernels of one-wavefront blocks that move 1-2 KiB each
 * 9-13 %, and buys nothing any more: large blocks, whose loads and stores run in separate runs (below),
 * measure the same at 8, 12 and 16.  (A block that streams a long slice alone on its compute unit moves
 * about 39 GB/s of payload whatever the depth: the unit keeps some 15 KiB of requests in flight.) */
#ifndef NVSHMEMI_AMD_COPY_DEEP_UNROLL
#define NVSHMEMI_AMD_COPY_DEEP_UNROLL 8
#endif
#ifndef NVSHMEMI_AMD_COPY_DEEP_MIN
#define NVSHMEMI_AMD_COPY_DEEP_MIN 32
#endif
/* Cache policy of the vector body.  Stores stream (non-temporal): a copy never reads its destination
 * back.  Loads stay cacheable for short and medium copies, because callers often push the same source
 * to several PEs (top-k token dispatch, all-push collectives) and the repeats then hit in L2 (measured
 * 1.4x on the MoE dispatch).  A long copy streams its loads too when the source cannot be expected in the
 * Infinity Cache: a put of NVSHMEMI_AMD_COPY_NT_BYTES (1 MiB) or more, or a get of NVSHMEMI_AMD_GET_NT_BYTES
 * (64 KiB) or more, whose size times the number of thread groups of its scope in the grid - what the grid
 * moves if every group copies as much - exceeds NVSHMEMI_AMD_COPY_CACHE_BYTES (256 MiB).  Shorter gets
 * always stream.  Measured on puts from 16 blocks per PE on 8 PEs:
 * +5 % at 256 MiB and +5.5 % at 64 MiB per PE with streamed loads, but 45 -> 86 us at 16 MiB and
 * 68 -> 118 us at 32 MiB per PE, sizes whose sources the cache holds from one put to the next.
 * NVSHMEMI_AMD_COPY_NT overrides the choice for a translation unit: bit 0 set = always non-temporal
 * loads, 0 = never; bit 1 = non-temporal stores. */
#ifndef NVSHMEMI_AMD_COPY_NT_BYTES
#define NVSHMEMI_AMD_COPY_NT_BYTES (1u << 20)
#endif
#ifndef NVSHMEMI_AMD_COPY_CACHE_BYTES
#define NVSHMEMI_AMD_COPY_CACHE_BYTES (256ull << 20)
#endif
#ifndef NVSHMEMI_AMD_GET_NT_BYTES /* gets shorter than this stream their loads without looking at the grid */
#define NVSHMEMI_AMD_GET_NT_BYTES (64u << 10)
#endif

/* A 16-byte store at agent scope (written through the L2).  The compiler has no such store, so it is
 * written as inline assembly, and the compiler does not know that the statement is a vector memory
 * store: it would not keep the one wait state this GPU needs between a store of more than 8 bytes
 * and a write to the registers that hold the store's data, so the s_nop supplies it (without it a
 * following address computation that reused the data registers corrupted the stored value). */
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_store16_agent(char *p, nvshmemi_v4u v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}

template <bool SRC_ALIGNED>
NVSHMEMI_DEVICE_INLINE nvshmemi_v4u nvshmemi_amd_load16(const char *p) {
    if (SRC_ALIGNED) return *reinterpret_cast<const nvshmemi_v4u *>(p);
    return *reinterpret_cast<const nvshmemi_v4u_unaligned *>(p);
}

template <bool SRC_ALIGNED, bool NT_LOAD>
NVSHMEMI_DEVICE_INLINE nvshmemi_v4u nvshmemi_amd_stream_load16(const char *p) {
    if (NT_LOAD && SRC_ALIGNED) return __builtin_nontemporal_load(reinterpret_cast<const nvshmemi_v4u *>(p));
    return nvshmemi_amd_load16<SRC_ALIGNED>(p);
}
/* Where the stores of a copy go: streamed (non-temporal; the lines stay dirty in this XCD's L2 until
 * they are evicted or a release writes the L2 back) or written through the L2 to memory at agent scope,
 * which leaves nothing for a later release to write back.  (Write-through as the default of plain
 * copies was measured too, as sc1 and as sc1 nt: +1.5 % when one-wavefront blocks fill the GPU, -3..4 %
 * for a few 1024-thread blocks per PE, so plain copies keep nt.) */
enum nvshmemi_amd_store_policy_t { NVSHMEMI_AMD_STORE_STREAM = 0, NVSHMEMI_AMD_STORE_WRITE_THROUGH = 1 };

template <int STORE = NVSHMEMI_AMD_STORE_STREAM>
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_stream_store16(char *p, nvshmemi_v4u v) {
    if (STORE == NVSHMEMI_AMD_STORE_WRITE_THROUGH) {
        // sc1 nt: written through at agent scope and marked streaming (+3 % over plain sc1 on the per-row
        // put_signal token dispatch); the s_nop for the same reason as in nvshmemi_amd_store16_agent
        asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
        return;
    }
#if defined(NVSHMEMI_AMD_COPY_NT) && !(NVSHMEMI_AMD_COPY_NT & 2)
    *reinterpret_cast<nvshmemi_v4u *>(p) = v;
#else
    __builtin_nontemporal_store(v, reinterpret_cast<nvshmemi_v4u *>(p));
#endif
}
template <int STORE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_store_byte(char *p, char v) {
    if (STORE == NVSHMEMI_AMD_STORE_WRITE_THROUGH)
        __hip_atomic_store(reinterpret_cast<unsigned char *>(p), (unsigned char)v, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    else
        *p = v;
}

/* Lane `tid` of `nthr` owns vectors tid, tid+nthr, ...  Rounds of U vectors per lane are straight-line
 * code - U independent loads issued before the first store - and run while the lane still has U
 * vectors left; with CASCADE the remainder is handled by the same code at U/2, U/4, ... 1, so a short
 * copy (a 14 KiB row moved by one wavefront is 14 vectors per lane: 4 + 4 + 4 + 2) keeps most of its
 * loads in flight.  No per-vector predicates: branches between the loads would make them wait for each
 * other. */
template <bool SRC_ALIGNED, bool NT_LOAD, int STORE, int U, bool CASCADE>
NVSHMEMI_DEVICE_INLINE size_t nvshmemi_amd_copy_rounds(char *__restrict__ dst,
                                                      const char *__restrict__ src, size_t nvec,
                                                      size_t i, size_t nthr) {
    for (; i + (U - 1) * nthr < nvec; i += U * nthr) {
        nvshmemi_v4u v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
            v[u] = nvshmemi_amd_stream_load16<SRC_ALIGNED, NT_LOAD>(src + 16 * (i + u * nthr));
#pragma unroll
        for (int u = 0; u < U; ++u) nvshmemi_amd_stream_store16<STORE>(dst + 16 * (i + u * nthr), v[u]);
    }
    /* next depth: half of a power of two, else the largest power of two below U (14 -> 8 -> 4 -> 2 -> 1) */
    constexpr int NEXT = (U & (U - 1)) ? (U >= 16 ? 16 : U >= 8 ? 8 : U >= 4 ? 4 : 2) : U / 2;
    if constexpr (CASCADE && U > 1)
        return nvshmemi_amd_copy_rounds<SRC_ALIGNED, NT_LOAD, STORE, NEXT, true>(dst, src, nvec, i, nthr);
    return i;
}

/* The translation unit's fixed choice for the loads of the ordinary rounds; the deep rounds of a long
 * copy choose at run time. */
#if defined(NVSHMEMI_AMD_COPY_NT) && (NVSHMEMI_AMD_COPY_NT & 1)
#define NVSHMEMI_AMD_COPY_NT_ALWAYS true
#else
#define NVSHMEMI_AMD_COPY_NT_ALWAYS false
#endif

/* Deep rounds of a long copy by whole wavefronts: per round the group moves U * nthr consecutive vectors
 * with U loads per lane issued back to back, then U stores.  All addresses are wave-uniform bases (scalar
 * registers) plus the lane's 16 * lane, so the U vectors in flight cost 4 U vector registers and no
 * address registers of their own (one address pair per vector made the compiler serialise the round to
 * stay within its register budget).  Returns the number of vectors moved, a multiple of U * nthr.
 *
 * Two layouts of a round:
 * - blocks of fewer than NVSHMEMI_AMD_COPY_PHASED_THREADS threads: wavefront w owns the U consecutive KiB
 *   [w * U, (w + 1) * U) of the round;
 * - larger blocks (block scope only): the u-th instruction of all wavefronts covers the nthr * 16
 *   consecutive bytes [u * nthr * 16, (u + 1) * nthr * 16), wavefront w its w-th KiB, so the block sweeps the
 *   round in address order, and the wavefronts stay in step: they meet after the loads of a round are
 *   issued and again after its stores are issued, so the compute unit's memory pipeline sees the round as
 *   one run of loads followed by one run of stores instead of the two interleaved.  Interleaved, the
 *   stores' acknowledgements take as long as the loads between them (L1-to-L2 write latency 950 cycles
 *   against 320 in runs) and fill the L1's store queue, which then holds up the loads behind it.  16 blocks
 *   of 1024 threads per PE move 4.73 TB/s interleaved, 5.56 in runs and 6.05 in runs swept in address order;
 *   one such block 61, 77 and 78 GB/s.  Blocks of 256 threads or fewer share their compute unit with other
 *   blocks, whose requests interleave anyway: neither the barriers nor the sweep changes their rate.  (The
 *   number of rounds is the same for every wavefront of the block, so all of them reach every barrier.) */
#ifndef NVSHMEMI_AMD_COPY_PHASED_THREADS
#define NVSHMEMI_AMD_COPY_PHASED_THREADS 512
#endif
template <bool NT_LOAD, int STORE, int U, bool BLOCK_WIDE>
NVSHMEMI_DEVICE_INLINE size_t nvshmemi_amd_copy_deep_rounds(char *__restrict__ dst, const char *__restrict__ src,
                                                           size_t nvec, unsigned tid, size_t nthr) {
    const size_t per_round = (size_t)U * nthr;
    const size_t rounds = nvec / per_round;
    const size_t wave = (size_t)__builtin_amdgcn_readfirstlane(tid >> 6);
    const unsigned lane_off = (tid & 63u) * 16u;
    const bool phased = BLOCK_WIDE && nthr >= NVSHMEMI_AMD_COPY_PHASED_THREADS;
    const size_t step = phased ? nthr * 16 : (size_t)1024;              /* from one instruction to the next */
    const size_t wave_off = wave * (phased ? (size_t)1024 : (size_t)(U * 1024));
    const char *s0 = src + wave_off;
    char *d0 = dst + wave_off;
    /* In the first layout the rounds are walked from a start that differs from block to block, wrapping at
     * the end.  Blocks that each stream a slice of one large message otherwise march in step, at equal
     * offsets in slices that lie a power of two (or the PE distance) apart, and keep meeting on the same
     * memory channels.  (The sweeping blocks do not gain from it, and lose 3 % on 4 MiB slices.) */
#ifndef NVSHMEMI_AMD_COPY_ROTATE
#define NVSHMEMI_AMD_COPY_ROTATE 1
#endif
    size_t r = 0;
    if (NVSHMEMI_AMD_COPY_ROTATE && !phased && rounds >= 8 && rounds <= 0xffffffffu) {
        const unsigned h = (blockIdx.x * 0x9E3779B1u) ^ (blockIdx.y * 0x85EBCA77u) ^ (blockIdx.z * 0xC2B2AE3Du);
        r = (size_t)(((uint64_t)h * (uint64_t)(rounds & 0xffffffffu)) >> 32);  /* in [0, rounds) */
    }
    for (size_t k = 0; k < rounds; ++k) {
        const char *s = s0 + r * (16 * per_round);
        char *d = d0 + r * (16 * per_round);
        if (++r == rounds) r = 0;
        nvshmemi_v4u v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = nvshmemi_amd_stream_load16<true, NT_LOAD>(s + u * step + lane_off);
        if (BLOCK_WIDE && phased) asm volatile("s_barrier" ::: "memory");
#pragma unroll
        for (int u = 0; u < U; ++u) nvshmemi_amd_stream_store16<STORE>(d + u * step + lane_off, v[u]);
        if (BLOCK_WIDE && phased) asm volatile("s_barrier" ::: "memory");
    }
    return rounds * per_round;
}

/* How a copy loads its source: by the size of the call (the policy above), or streamed also when it is
 * short.  A get streams: its source is another PE's memory, which the caller reads once (the token combine,
 * 2 KiB per call from scattered rows: 5.73 -> 6.02 TB/s), whereas the source of a put is local data that is
 * often sent to several PEs.  Gets of 64 KiB or more follow the policy above like long puts. */
enum nvshmemi_amd_load_policy_t { NVSHMEMI_AMD_LOAD_BY_SIZE = 0, NVSHMEMI_AMD_LOAD_STREAM = 1 };

template <bool SRC_ALIGNED, int STORE, int LOAD = NVSHMEMI_AMD_LOAD_BY_SIZE, bool BLOCK_WIDE = false>
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_copy_vectors(char *__restrict__ dst,
                                                     const char *__restrict__ src, size_t nvec,
                                                     size_t tid, size_t nthr, bool stream_loads) {
#if NVSHMEMI_AMD_COPY_DEEP_UNROLL > NVSHMEMI_AMD_COPY_UNROLL
    /* (the second bound follows from the first for whole wavefronts; spelled out, it lets the compiler drop
     * the deep rounds and their registers where the caller's length is known to be short) */
    if (SRC_ALIGNED && (nthr & 63) == 0 && nvec >= (size_t)NVSHMEMI_AMD_COPY_DEEP_MIN * nthr &&
        nvec >= (size_t)NVSHMEMI_AMD_COPY_DEEP_MIN * 64) {
        const size_t done =
            stream_loads ? nvshmemi_amd_copy_deep_rounds<true, STORE, NVSHMEMI_AMD_COPY_DEEP_UNROLL, BLOCK_WIDE>(
                               dst, src, nvec, (unsigned)tid, nthr)
                         : nvshmemi_amd_copy_deep_rounds<false, STORE, NVSHMEMI_AMD_COPY_DEEP_UNROLL, BLOCK_WIDE>(
                               dst, src, nvec, (unsigned)tid, nthr);
        dst += 16 * done;
        src += 16 * done;
        nvec -= done;
    }
#endif
    if (LOAD == NVSHMEMI_AMD_LOAD_STREAM && !NVSHMEMI_AMD_COPY_NT_ALWAYS && !stream_loads)
        nvshmemi_amd_copy_rounds<SRC_ALIGNED, false, STORE, NVSHMEMI_AMD_COPY_UNROLL, true>(dst, src, nvec, tid, nthr);
    else
        nvshmemi_amd_copy_rounds<SRC_ALIGNED, NVSHMEMI_AMD_COPY_NT_ALWAYS || LOAD == NVSHMEMI_AMD_LOAD_STREAM, STORE,
                                 NVSHMEMI_AMD_COPY_UNROLL, true>(dst, src, nvec, tid, nthr);
}

template <int SCOPE, int STORE = NVSHMEMI_AMD_STORE_STREAM, int LOAD = NVSHMEMI_AMD_LOAD_BY_SIZE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_memcpy_threadgroup(void *__restrict__ dst_v,
                                                       const void *__restrict__ src_v, size_t len) {
    char *dst = static_cast<char *>(dst_v);
    const char *src = static_cast<const char *>(src_v);
    const size_t tid = (size_t)nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const size_t nthr = (size_t)nvshmemi_threadgroup_size<SCOPE>();
#if defined(NVSHMEMI_AMD_COPY_NT)
    const bool stream_loads = (NVSHMEMI_AMD_COPY_NT & 1) != 0;
#else
    /* (short copies decide without reading the launch dimensions: puts keep their loads cacheable, gets
     * stream) */
    bool stream_loads = LOAD == NVSHMEMI_AMD_LOAD_STREAM;
    if (len >= (LOAD == NVSHMEMI_AMD_LOAD_STREAM ? NVSHMEMI_AMD_GET_NT_BYTES : NVSHMEMI_AMD_COPY_NT_BYTES)) {
        const float per_block = SCOPE == NVSHMEMI_THREADGROUP_BLOCK ? 1.0f
                                : (float)(blockDim.x * blockDim.y * blockDim.z) /
                                      (SCOPE == NVSHMEMI_THREADGROUP_WARP ? (float)NVSHMEMI_WARP_SIZE : 1.0f);
        const float groups = (float)gridDim.x * (float)gridDim.y * (float)gridDim.z * per_block;
        stream_loads = (float)len * groups > (float)NVSHMEMI_AMD_COPY_CACHE_BYTES;
    } else if (LOAD == NVSHMEMI_AMD_LOAD_BY_SIZE) {
        stream_loads = false;
    }
#endif

    size_t head = (size_t)(-(uintptr_t)dst & 15);
    if (head > len) head = len;
    for (size_t i = tid; i < head; i += nthr) nvshmemi_amd_store_byte<STORE>(dst + i, src[i]);
    dst += head;
    src += head;
    len -= head;

    const size_t nvec = len / 16;
    if (nvec) {
        /* Long copies: the first lanes move the vectors in front of the next 1 KiB boundary of dst, so
         * that every wavefront access of the body is one aligned 1 KiB piece (HBM serves those
         * measurably faster than pieces that straddle the boundary). */
        size_t pre = 0;
        if (nvec >= 256) {
            pre = (size_t)((-(uintptr_t)dst >> 4) & 63);
            if (((uintptr_t)src & 15) == 0) nvshmemi_amd_copy_vectors<true, STORE, LOAD>(dst, src, pre, tid, nthr, stream_loads);
            else nvshmemi_amd_copy_vectors<false, STORE, LOAD>(dst, src, pre, tid, nthr, stream_loads);
        }
        constexpr bool block_wide = SCOPE == NVSHMEMI_THREADGROUP_BLOCK;   // every wavefront of the block is here
        if (((uintptr_t)src & 15) == 0)
            nvshmemi_amd_copy_vectors<true, STORE, LOAD, block_wide>(dst + 16 * pre, src + 16 * pre, nvec - pre, tid, nthr, stream_loads);
        else
            nvshmemi_amd_copy_vectors<false, STORE, LOAD, block_wide>(dst + 16 * pre, src + 16 * pre, nvec - pre, tid, nthr, stream_loads);
    }
    const size_t done = nvec * 16;
    for (size_t i = done + tid; i < len; i += nthr) nvshmemi_amd_store_byte<STORE>(dst + i, src[i]);
}

/* ------------------------------------------------------------------------------------------------
 * put / get / p / g  (reference common/nvshmemi_common_device.cuh:396-505)
 * The non-blocking forms are the same code on a load/store path, as in the reference (:410-427).
 * ---------------------------------------------------------------------------------------------- */
template <typename T, int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_put(T *dest, const T *source, size_t nelems, int pe) {
    nvshmemi_threadgroup_sync<SCOPE>();
    nvshmemi_memcpy_threadgroup<SCOPE>(nvshmemi_amd_remote(dest, pe), nvshmemi_amd_local(source),
                                       nelems * sizeof(T));
    nvshmemi_threadgroup_sync<SCOPE>();
}

template <typename T, int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_get(T *dest, const T *source, size_t nelems, int pe) {
    nvshmemi_threadgroup_sync<SCOPE>();
    nvshmemi_memcpy_threadgroup<SCOPE, NVSHMEMI_AMD_STORE_STREAM, NVSHMEMI_AMD_LOAD_STREAM>(
        nvshmemi_amd_local(dest), nvshmemi_amd_remote(source, pe), nelems * sizeof(T));
    nvshmemi_threadgroup_sync<SCOPE>();
}

/* The value is stored with an agent-scope atomic store of its bits, so that it leaves this XCD's L2
 * on its own: the OpenSHMEM idiom "p a flag, the target waits on it" must make progress without a
 * quiet in between. */
template <typename T>
NVSHMEMI_DEVICE_INLINE void nvshmemi_p(T *dest, const T value, int pe) {
    char *p = nvshmemi_amd_remote(dest, pe);
    if constexpr (sizeof(T) == 1) {
        uint8_t v;
        __builtin_memcpy(&v, &value, 1);
        __hip_atomic_store((uint8_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if constexpr (sizeof(T) == 2) {
        uint16_t v;
        __builtin_memcpy(&v, &value, 2);
        __hip_atomic_store((uint16_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if constexpr (sizeof(T) == 4) {
        uint32_t v;
        __builtin_memcpy(&v, &value, 4);
        __hip_atomic_store((uint32_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        static_assert(sizeof(T) == 8, "scalar put supports 1, 2, 4 and 8 byte elements");
        uint64_t v;
        __builtin_memcpy(&v, &value, 8);
        __hip_atomic_store((uint64_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

/* A remote word may be written by another PE while this kernel runs, so the read is an agent-scope
 * atomic load of the element's bits (never kept in a register, never served from a stale line). */
template <typename T>
NVSHMEMI_DEVICE_INLINE T nvshmemi_g(const T *source, int pe) {
    const char *p = nvshmemi_amd_remote(source, pe);
    T out;
    if constexpr (sizeof(T) == 1) {
        uint8_t v = __hip_atomic_load((const uint8_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_memcpy(&out, &v, 1);
    } else if constexpr (sizeof(T) == 2) {
        uint16_t v = __hip_atomic_load((const uint16_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_memcpy(&out, &v, 2);
    } else if constexpr (sizeof(T) == 4) {
        uint32_t v = __hip_atomic_load((const uint32_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_memcpy(&out, &v, 4);
    } else {
        static_assert(sizeof(T) == 8, "scalar get supports 1, 2, 4 and 8 byte elements");
        uint64_t v = __hip_atomic_load((const uint64_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_memcpy(&out, &v, 8);
    }
    return out;
}

/* Strided forms (reference src/include/device/nvshmem_defines.h:345-431): element i of the source
 * at stride sst goes to element i*dst of the destination. */
template <typename T, int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_iput(T *dest, const T *source, ptrdiff_t dst, ptrdiff_t sst,
                                          size_t nelems, int pe) {
    nvshmemi_threadgroup_sync<SCOPE>();
    T *d = reinterpret_cast<T *>(nvshmemi_amd_remote(dest, pe));
    const T *s = reinterpret_cast<const T *>(nvshmemi_amd_local(source));
    const size_t tid = (size_t)nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const size_t nthr = (size_t)nvshmemi_threadgroup_size<SCOPE>();
    for (size_t i = tid; i < nelems; i += nthr) d[(ptrdiff_t)i * dst] = s[(ptrdiff_t)i * sst];
    nvshmemi_threadgroup_sync<SCOPE>();
}

template <typename T, int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_iget(T *dest, const T *source, ptrdiff_t dst, ptrdiff_t sst,
                                          size_t nelems, int pe) {
    nvshmemi_threadgroup_sync<SCOPE>();
    T *d = reinterpret_cast<T *>(nvshmemi_amd_local(dest));
    const T *s = reinterpret_cast<const T *>(nvshmemi_amd_remote(source, pe));
    const size_t tid = (size_t)nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const size_t nthr = (size_t)nvshmemi_threadgroup_size<SCOPE>();
    for (size_t i = tid; i < nelems; i += nthr) d[(ptrdiff_t)i * dst] = s[(ptrdiff_t)i * sst];
    nvshmemi_threadgroup_sync<SCOPE>();
}

/* ------------------------------------------------------------------------------------------------
 * quiet / fence  (reference common/nvshmemi_common_device.cuh:352-385): one GPU, so agent scope.
 * ---------------------------------------------------------------------------------------------- */
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_quiet() {
    nvshmemi_amd_wait_vm();
    nvshmemi_threadgroup_sync<SCOPE>();
    if (nvshmemi_thread_id_in_threadgroup<SCOPE>() == 0)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    nvshmemi_threadgroup_sync<SCOPE>();
}

/* ------------------------------------------------------------------------------------------------
 * signal / put_signal  (reference common/nvshmemi_common_device.cuh:507-561)
 * ---------------------------------------------------------------------------------------------- */
NVSHMEMI_DEVICE_INLINE void nvshmemi_signal_op(uint64_t *sig_addr, uint64_t signal, int sig_op,
                                               int pe) {
    uint64_t *p = reinterpret_cast<uint64_t *>(nvshmemi_amd_remote(sig_addr, pe));
    if ((sig_op & NVSHMEMI_AMD_SIGNAL_OP_MASK) == NVSHMEM_SIGNAL_SET)
        __hip_atomic_store(p, signal, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        __hip_atomic_fetch_add(p, signal, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* The signal of a put-with-signal publishes the data that the group wrote before it. */
NVSHMEMI_DEVICE_INLINE void nvshmemi_signal_op_release(uint64_t *sig_addr, uint64_t signal,
                                                       int sig_op, int pe) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    nvshmemi_signal_op(sig_addr, signal, sig_op, pe);
}

/* put-with-signal.  Two orderings, chosen by the caller through sig_op:
 *  - default, the reference's (a full fence in front of the signal,
 *    common/nvshmemi_common_device.cuh:541-545): the payload streams into the L2, every wavefront waits
 *    for its stores, and the one lane that signals first releases at agent scope, which writes the
 *    XCD's L2 back - the payload and whatever else the group wrote before the call (a ring allreduce
 *    that accumulates into its destination with plain stores and is overwritten by a neighbour later
 *    relies on that);
 *  - NVSHMEMX_AMD_SIGNAL_PAYLOAD_ONLY, OpenSHMEM's: the payload is written through the L2 with
 *    agent-scope stores, so it is in memory once every wavefront has counted its stores down, and the
 *    signal follows with no fence at all.  An L2 write-back walks the whole L2, the write-backs of an
 *    XCD run one after the other, dirty lines leave at about 60 GB/s per XCD and other traffic crawls
 *    meanwhile: a token dispatch that signals each 14 KiB row took 17-24 ms with a release per row
 *    (whether the payload was streamed or written through, and also when the wavefronts of an XCD
 *    shared write-backs through a ticket lock: a write-back under that load takes some 20 us), against
 *    1.7 ms with one release per block.  Without the fence the per-row form takes a few ms.
 *    The library-wide option NVSHMEMI_AMD_OPTION_PUT_SIGNAL_PAYLOAD_ONLY (set from the environment or by
 *    nvshmemx_amd_set_put_signal_order) selects this order for every call, for programs that cannot
 *    edit their call sites. */
template <typename T, int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_put_signal(T *dest, const T *source, size_t nelems,
                                                uint64_t *sig_addr, uint64_t signal, int sig_op,
                                                int pe) {
    nvshmemi_threadgroup_sync<SCOPE>();
    if ((sig_op & NVSHMEMX_AMD_SIGNAL_PAYLOAD_ONLY) ||
        (nvshmemi_device_state_d.options & NVSHMEMI_AMD_OPTION_PUT_SIGNAL_PAYLOAD_ONLY)) {
        nvshmemi_memcpy_threadgroup<SCOPE, NVSHMEMI_AMD_STORE_WRITE_THROUGH>(
            nvshmemi_amd_remote(dest, pe), nvshmemi_amd_local(source), nelems * sizeof(T));
        nvshmemi_amd_wait_vm();
        nvshmemi_threadgroup_sync<SCOPE>();
        if (nvshmemi_thread_id_in_threadgroup<SCOPE>() == 0) nvshmemi_signal_op(sig_addr, signal, sig_op, pe);
    } else {
        nvshmemi_memcpy_threadgroup<SCOPE>(nvshmemi_amd_remote(dest, pe), nvshmemi_amd_local(source),
                                           nelems * sizeof(T));
        nvshmemi_amd_wait_vm();
        nvshmemi_threadgroup_sync<SCOPE>();
        if (nvshmemi_thread_id_in_threadgroup<SCOPE>() == 0)
            nvshmemi_signal_op_release(sig_addr, signal, sig_op, pe);
    }
    nvshmemi_threadgroup_sync<SCOPE>();
}

/* ------------------------------------------------------------------------------------------------
 * wait / test  (reference wait/nvshmemi_wait_until_apis.cuh:37-155, nvshmemi_test
 * common/nvshmemi_common_device.cuh:130-147)
 * ---------------------------------------------------------------------------------------------- */
template <typename T>
NVSHMEMI_DEVICE_INLINE bool nvshmemi_amd_compare(T found, int cmp, T expected) {
    switch (cmp) {
        case NVSHMEM_CMP_EQ: return found == expected;
        case NVSHMEM_CMP_NE: return found != expected;
        case NVSHMEM_CMP_GT: return found > expected;
        case NVSHMEM_CMP_LE: return found <= expected;
        case NVSHMEM_CMP_LT: return found < expected;
        case NVSHMEM_CMP_GE: return found >= expected;
        default: return true; /* an unknown comparator never blocks */
    }
}

template <typename T>
NVSHMEMI_DEVICE_INLINE T nvshmemi_amd_poll(const T *addr) {
    return __hip_atomic_load(addr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_record_timeout(const void *addr, uint64_t found,
                                                        uint64_t expected) {
    uint64_t *rec = reinterpret_cast<uint64_t *>(
        nvshmemi_amd_remote(nvshmemi_device_state_d.timeout_record, nvshmemi_amd_my_pe()));
    /* the count the host checks at its synchronisation points; the record's first word is this timeout's
     * number in that count (never 0), so that a report can tell a record of its own period from an older one */
    const uint64_t seq = __hip_atomic_fetch_add(nvshmemi_device_state_d.runtime_words + NVSHMEMI_AMD_TIMEOUT_COUNT_WORD,
                                                (uint64_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
    rec[1] = (uint64_t)(uintptr_t)addr;
    rec[2] = found;
    rec[3] = expected;
    __hip_atomic_store(rec, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    /* the host's copy of "something happened": any number of this period differs from what the host saw last */
    if (nvshmemi_device_state_d.timeout_flag)
        __hip_atomic_store(nvshmemi_device_state_d.timeout_flag, seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

/* Spin until `*ivar cmp value`; `ivar` is a local operand.  Returns the value that ended the wait.
 * The final acquire makes data published before the signal visible to the caller; the reference's
 * typed waits fence the same way (__threadfence via nvshmemi_transfer_syncapi_update_mem). */
template <typename T, bool ACQUIRE = true>
NVSHMEMI_DEVICE_INLINE T nvshmemi_wait_until(T *ivar, int cmp, T value) {
    const T *addr = reinterpret_cast<const T *>(nvshmemi_amd_local(ivar));
    const uint64_t limit = nvshmemi_device_state_d.spin_limit;
    uint64_t polls = 0;
    T found = nvshmemi_amd_poll(addr);
    while (!nvshmemi_amd_compare(found, cmp, value)) {
        if (limit && ++polls > limit) {
            nvshmemi_amd_record_timeout(addr, (uint64_t)found, (uint64_t)value);
            break;
        }
        __builtin_amdgcn_s_sleep(1);
        found = nvshmemi_amd_poll(addr);
    }
    /* (a caller that waits for several variables in a row asks for no fence and issues one itself) */
    if (ACQUIRE) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return found;
}

template <typename T>
NVSHMEMI_DEVICE_INLINE int nvshmemi_test(T *ivar, int cmp, T value) {
    const T *addr = reinterpret_cast<const T *>(nvshmemi_amd_local(ivar));
    if (nvshmemi_amd_compare(nvshmemi_amd_poll(addr), cmp, value)) {
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        return 1;
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------------
 * Waits and tests over sets of variables (reference src/include/device/nvshmem_defines.h:446-735).
 * status[i] != 0 takes ivars[i] out of the set; `values` is one comparison value (VECTOR false)
 * or one per variable.  The "any" forms return an index that satisfies the comparison, or SIZE_MAX
 * for an empty set; the "some" forms store the satisfied indices and return their number, at least
 * one unless the set is empty.  The reference starts its "any" scans at a rotating index; here a
 * scan starts at 0, which returns a member of the same set of valid answers.  A wait that exceeds
 * the spin limit is recorded like in nvshmemi_wait_until and returns SIZE_MAX / 0.
 * ---------------------------------------------------------------------------------------------- */
template <typename T, bool VECTOR>
NVSHMEMI_DEVICE_INLINE T nvshmemi_amd_cmp_value(const T *values, size_t i) {
    return VECTOR ? values[i] : values[0];
}
template <typename T, bool VECTOR>
NVSHMEMI_DEVICE_INLINE void nvshmemi_wait_until_all(T *ivars, size_t nelems, const int *status, int cmp,
                                                    const T *values) {
    /* Eight variables are polled per memory round trip and the front of the set moves past those
     * that are satisfied; one acquire at the end covers them all.  (One wait after the other costs a
     * round trip and a fence per variable even when everything has arrived: 8 variables 2.9 us.) */
    if (nelems == 0) return;
    const T *addr = reinterpret_cast<const T *>(nvshmemi_amd_local(ivars));
    const uint64_t limit = nvshmemi_device_state_d.spin_limit;
    uint64_t sweeps = 0;
    size_t first = 0;
    while (first < nelems) {
        T x[8];
#pragma unroll
        for (size_t k = 0; k < 8; ++k) x[k] = nvshmemi_amd_poll(addr + (first + k < nelems ? first + k : nelems - 1));
        size_t ok = 0;
#pragma unroll
        for (size_t k = 0; k < 8; ++k) {
            const size_t i = first + k;
            if (ok == k && i < nelems &&
                ((status && status[i]) || nvshmemi_amd_compare(x[k], cmp, nvshmemi_amd_cmp_value<T, VECTOR>(values, i))))
                ++ok;
        }
        first += ok;
        if (ok == 8 || first >= nelems) continue;
        if (limit && ++sweeps > limit) {
            nvshmemi_amd_record_timeout(addr + first, (uint64_t)x[ok], (uint64_t)nvshmemi_amd_cmp_value<T, VECTOR>(values, first));
            break;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}
/* One pass over the set, eight variables per memory round trip: visit(i, satisfied) is called for the
 * members in index order until it returns false.  The caller acquires once if it reports success. */
template <typename T, bool VECTOR, typename Visit>
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_scan_set(T *ivars, size_t nelems, const int *status, int cmp,
                                                  const T *values, Visit visit) {
    if (nelems == 0) return;
    const T *addr = reinterpret_cast<const T *>(nvshmemi_amd_local(ivars));
    for (size_t first = 0; first < nelems; first += 8) {
        T x[8];
#pragma unroll
        for (size_t k = 0; k < 8; ++k) x[k] = nvshmemi_amd_poll(addr + (first + k < nelems ? first + k : nelems - 1));
#pragma unroll
        for (size_t k = 0; k < 8; ++k) {
            const size_t i = first + k;
            if (i >= nelems) return;
            if (status && status[i]) continue;
            if (!visit(i, nvshmemi_amd_compare(x[k], cmp, nvshmemi_amd_cmp_value<T, VECTOR>(values, i)))) return;
        }
    }
}
template <typename T, bool VECTOR>
NVSHMEMI_DEVICE_INLINE int nvshmemi_test_all(T *ivars, size_t nelems, const int *status, int cmp,
                                             const T *values) {
    bool all = true;
    nvshmemi_amd_scan_set<T, VECTOR>(ivars, nelems, status, cmp, values, [&](size_t, bool ok) {
        all = ok;
        return ok;
    });
    if (all) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return all ? 1 : 0;
}
template <typename T, bool VECTOR>
NVSHMEMI_DEVICE_INLINE size_t nvshmemi_test_any(T *ivars, size_t nelems, const int *status, int cmp,
                                                const T *values) {
    size_t hit = SIZE_MAX;
    nvshmemi_amd_scan_set<T, VECTOR>(ivars, nelems, status, cmp, values, [&](size_t i, bool ok) {
        if (ok) hit = i;
        return !ok;
    });
    if (hit != SIZE_MAX) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return hit;
}
template <typename T, bool VECTOR>
NVSHMEMI_DEVICE_INLINE size_t nvshmemi_test_some(T *ivars, size_t nelems, size_t *indices, const int *status,
                                                 int cmp, const T *values) {
    size_t found = 0;
    nvshmemi_amd_scan_set<T, VECTOR>(ivars, nelems, status, cmp, values, [&](size_t i, bool ok) {
        if (ok) indices[found++] = i;
        return true;
    });
    if (found) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return found;
}
template <typename T, bool VECTOR>
NVSHMEMI_DEVICE_INLINE size_t nvshmemi_wait_until_any(T *ivars, size_t nelems, const int *status, int cmp,
                                                      const T *values) {
    bool empty = true;
    for (size_t i = 0; i < nelems && empty; ++i) empty = status && status[i];
    if (empty) return SIZE_MAX;
    const uint64_t limit = nvshmemi_device_state_d.spin_limit;
    for (uint64_t sweeps = 0;; ++sweeps) {
        const size_t hit = nvshmemi_test_any<T, VECTOR>(ivars, nelems, status, cmp, values);
        if (hit != SIZE_MAX) return hit;
        if (limit && sweeps >= limit) {
            nvshmemi_amd_record_timeout(ivars, 0, (uint64_t)values[0]);
            return SIZE_MAX;
        }
        __builtin_amdgcn_s_sleep(1);
    }
}
template <typename T, bool VECTOR>
NVSHMEMI_DEVICE_INLINE size_t nvshmemi_wait_until_some(T *ivars, size_t nelems, size_t *indices,
                                                       const int *status, int cmp, const T *values) {
    size_t found = nvshmemi_test_some<T, VECTOR>(ivars, nelems, indices, status, cmp, values);
    if (found) return found;
    const size_t hit = nvshmemi_wait_until_any<T, VECTOR>(ivars, nelems, status, cmp, values);
    if (hit == SIZE_MAX) return 0;
    indices[0] = hit;
    return 1;
}

/* ------------------------------------------------------------------------------------------------
 * Atomic memory operations (reference src/include/device/nvshmem_defines.h:742-1236, whose
 * load/store branch applies atomic*_system to the translated address).  Here: relaxed agent-scope
 * atomics on the target PE's copy; every operation works at the full width of its type (the
 * reference narrows a few through its sub-type casts, e.g. ulong fetch_add through unsigned int,
 * and leaves longlong / int64 / ptrdiff add and inc out).  float and double go through an integer
 * exchange / load / store of the same width.
 * ---------------------------------------------------------------------------------------------- */
template <typename T> struct nvshmemi_amd_amo_word { typedef T type; };
template <> struct nvshmemi_amd_amo_word<float> { typedef uint32_t type; };
template <> struct nvshmemi_amd_amo_word<double> { typedef uint64_t type; };

template <typename T>
NVSHMEMI_DEVICE_INLINE typename nvshmemi_amd_amo_word<T>::type nvshmemi_amd_amo_bits(T v) {
    typename nvshmemi_amd_amo_word<T>::type w;
    __builtin_memcpy(&w, &v, sizeof w);
    return w;
}
template <typename T>
NVSHMEMI_DEVICE_INLINE T nvshmemi_amd_amo_value(typename nvshmemi_amd_amo_word<T>::type w) {
    T v;
    __builtin_memcpy(&v, &w, sizeof v);
    return v;
}
template <typename T>
NVSHMEMI_DEVICE_INLINE typename nvshmemi_amd_amo_word<T>::type *nvshmemi_amd_amo_target(const T *target, int pe) {
    return reinterpret_cast<typename nvshmemi_amd_amo_word<T>::type *>(
        nvshmemi_amd_remote(const_cast<T *>(target), pe));
}

template <typename T>
NVSHMEMI_DEVICE_INLINE T nvshmemi_atomic_fetch(const T *target, int pe) {
    return nvshmemi_amd_amo_value<T>(
        __hip_atomic_load(nvshmemi_amd_amo_target(target, pe), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
template <typename T>
NVSHMEMI_DEVICE_INLINE void nvshmemi_atomic_set(T *target, T value, int pe) {
    __hip_atomic_store(nvshmemi_amd_amo_target(target, pe), nvshmemi_amd_amo_bits(value), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
NVSHMEMI_DEVICE_INLINE T nvshmemi_atomic_swap(T *target, T value, int pe) {
    return nvshmemi_amd_amo_value<T>(__hip_atomic_exchange(nvshmemi_amd_amo_target(target, pe),
                                                          nvshmemi_amd_amo_bits(value), __ATOMIC_RELAXED,
                                                          __HIP_MEMORY_SCOPE_AGENT));
}
/* if (*target == cond) *target = value; returns the value found */
template <typename T>
NVSHMEMI_DEVICE_INLINE T nvshmemi_atomic_compare_swap(T *target, T cond, T value, int pe) {
    T expected = cond;
    __hip_atomic_compare_exchange_strong(nvshmemi_amd_amo_target(target, pe), &expected, value,
                                         __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return expected;
}
template <typename T>
NVSHMEMI_DEVICE_INLINE T nvshmemi_atomic_fetch_add(T *target, T value, int pe) {
    return __hip_atomic_fetch_add(nvshmemi_amd_amo_target(target, pe), value, __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
NVSHMEMI_DEVICE_INLINE T nvshmemi_atomic_fetch_and(T *target, T value, int pe) {
    return __hip_atomic_fetch_and(nvshmemi_amd_amo_target(target, pe), value, __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
NVSHMEMI_DEVICE_INLINE T nvshmemi_atomic_fetch_or(T *target, T value, int pe) {
    return __hip_atomic_fetch_or(nvshmemi_amd_amo_target(target, pe), value, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
NVSHMEMI_DEVICE_INLINE T nvshmemi_atomic_fetch_xor(T *target, T value, int pe) {
    return __hip_atomic_fetch_xor(nvshmemi_amd_amo_target(target, pe), value, __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_AGENT);
}

/* ------------------------------------------------------------------------------------------------
 * Teams (reference non_abi/device/team/nvshmemi_team_defines.cuh:95-141).  A team is the strided
 * PE set {start + i*stride, i < size}; the table holds every team as each PE sees it.
 * ---------------------------------------------------------------------------------------------- */
NVSHMEMI_DEVICE_INLINE nvshmemi_amd_team_view_t nvshmemi_amd_team_view_of(nvshmem_team_t team, int pe) {
    nvshmemi_amd_team_view_t v;
    if (team == NVSHMEM_TEAM_WORLD) {
        v.start = 0; v.stride = 1; v.size = nvshmemi_device_state_d.npes; v.my_pe = pe;
    } else if (team < 0 || team >= NVSHMEMI_AMD_MAX_TEAMS) {
        v.start = 0; v.stride = 1; v.size = 0; v.my_pe = -1;
    } else {
        v = nvshmemi_device_state_d.team_views[team * NVSHMEMI_AMD_MAX_PES + pe];
    }
    return v;
}
NVSHMEMI_DEVICE_INLINE nvshmemi_amd_team_view_t nvshmemi_amd_team_view(nvshmem_team_t team) {
    return nvshmemi_amd_team_view_of(team, nvshmemi_amd_my_pe());
}
/* world PE of member `idx` */
NVSHMEMI_DEVICE_INLINE int nvshmemi_amd_team_pe(const nvshmemi_amd_team_view_t &v, int idx) {
    return v.start + idx * v.stride;
}
NVSHMEMI_DEVICE_INLINE int nvshmemi_team_my_pe(nvshmem_team_t team) {
    const nvshmemi_amd_team_view_t v = nvshmemi_amd_team_view(team);
    return v.size > 0 ? v.my_pe : -1;
}
NVSHMEMI_DEVICE_INLINE int nvshmemi_team_n_pes(nvshmem_team_t team) {
    const nvshmemi_amd_team_view_t v = nvshmemi_amd_team_view(team);
    return v.size > 0 ? v.size : -1;
}
/* Member src_pe of src_team as an index of dest_team, or -1; an index equal to the size wraps to
 * member 0 and larger ones give -1, as in the reference (nvshmemi_team_defines.cuh:120-141). */
NVSHMEMI_DEVICE_INLINE int nvshmemi_team_translate_pe(nvshmem_team_t src_team, int src_pe,
                                                      nvshmem_team_t dest_team) {
    const nvshmemi_amd_team_view_t s = nvshmemi_amd_team_view(src_team);
    const nvshmemi_amd_team_view_t d = nvshmemi_amd_team_view(dest_team);
    if (s.size <= 0 || d.size <= 0 || src_pe < 0 || src_pe > s.size) return -1;
    const int off = nvshmemi_amd_team_pe(s, src_pe % s.size) - d.start;
    if (off < 0 || off % d.stride != 0 || off / d.stride >= d.size) return -1;
    return off / d.stride;
}
/* arrival words of PE `pe` for `team`, and that PE's epoch word */
NVSHMEMI_DEVICE_INLINE uint64_t *nvshmemi_amd_sync_row(nvshmem_team_t team, int pe) {
    if (team == NVSHMEM_TEAM_WORLD)
        return reinterpret_cast<uint64_t *>(nvshmemi_amd_remote(nvshmemi_device_state_d.sync_flags, pe));
    return nvshmemi_device_state_d.team_sync +
           ((size_t)team * NVSHMEMI_AMD_MAX_PES + (size_t)pe) * NVSHMEMI_AMD_TEAM_SYNC_WORDS;
}
NVSHMEMI_DEVICE_INLINE uint64_t *nvshmemi_amd_sync_epoch(nvshmem_team_t team, int pe) {
    if (team == NVSHMEM_TEAM_WORLD)
        return reinterpret_cast<uint64_t *>(nvshmemi_amd_remote(nvshmemi_device_state_d.sync_epoch, pe));
    return nvshmemi_amd_sync_row(team, pe) + NVSHMEMI_AMD_MAX_PES;
}

/* ------------------------------------------------------------------------------------------------
 * barrier / sync  (reference coll/barrier.cuh:24-251, coll/utils.cuh:38-51)
 *
 * One thread group per PE takes part.  Flat exchange (the reference's dissemination with radix =
 * team size, its choice for block scope on a load/store path, barrier.cuh:195-225): PE me stores
 * its new epoch into word [me] of every PE's flag row, then waits until all npes words of its own
 * row have reached that epoch.  Epochs only grow, so rows are never reset.
 * ---------------------------------------------------------------------------------------------- */
/* The second half of a synchronisation whose number - the PE's count of synchronisations on the team
 * so far, plus one - the caller has read already (after a thread group sync of its own): records it,
 * tells every member and waits for all of them. */
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_sync_arrive_wait(nvshmem_team_t team, const nvshmemi_amd_team_view_t &v,
                                                          uint64_t epoch) {
    const int me = nvshmemi_amd_my_pe();
    const int tid = nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const int nthr = nvshmemi_threadgroup_size<SCOPE>();
    nvshmemi_threadgroup_sync<SCOPE>();
    if (tid == 0) *reinterpret_cast<volatile uint64_t *>(nvshmemi_amd_sync_epoch(team, me)) = epoch;
    /* one release in front of a lane's arrival stores and one acquire behind its waits, however many
     * members the lane serves (a single thread serves them all: 8 PEs in 2.2 us instead of 3.8 us) */
    if (tid < v.size) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    for (int i = tid; i < v.size; i += nthr) {
        uint64_t *flag = nvshmemi_amd_sync_row(team, nvshmemi_amd_team_pe(v, i)) + v.my_pe;
        __hip_atomic_store(flag, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    uint64_t *row = nvshmemi_amd_sync_row(team, me);
    if (nthr >= v.size) {
        if (tid < v.size) nvshmemi_wait_until<uint64_t, false>(row + tid, NVSHMEM_CMP_GE, epoch);
    } else {
        /* a lane that serves several members polls eight of their words per round trip */
        const uint64_t *words = reinterpret_cast<const uint64_t *>(nvshmemi_amd_local(row));
        const uint64_t limit = nvshmemi_device_state_d.spin_limit;
        uint64_t polls = 0;
        for (;;) {
            uint64_t lowest = ~(uint64_t)0;
            for (int i0 = tid; i0 < v.size; i0 += 8 * nthr) {
                uint64_t x[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int i = i0 + k * nthr;
                    x[k] = nvshmemi_amd_poll(words + (i < v.size ? i : i0));
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) lowest = x[k] < lowest ? x[k] : lowest;
            }
            if (lowest >= epoch) break;
            if (limit && ++polls > limit) {
                nvshmemi_amd_record_timeout(words + tid, lowest, epoch);
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
    }
    if (tid < v.size) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    nvshmemi_threadgroup_sync<SCOPE>();
}

template <int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_sync_threadgroup(nvshmem_team_t team = NVSHMEM_TEAM_WORLD) {
    const int me = nvshmemi_amd_my_pe();
    const nvshmemi_amd_team_view_t v = nvshmemi_amd_team_view(team);
    if (v.size <= 0) return; /* not a member */
    nvshmemi_threadgroup_sync<SCOPE>();
    const uint64_t epoch = *reinterpret_cast<volatile uint64_t *>(nvshmemi_amd_sync_epoch(team, me)) + 1;
    nvshmemi_amd_sync_arrive_wait<SCOPE>(team, v, epoch);
}

template <int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_barrier_threadgroup(nvshmem_team_t team = NVSHMEM_TEAM_WORLD) {
    nvshmemi_quiet<SCOPE>();
    nvshmemi_sync_threadgroup<SCOPE>(team);
}

/* Barrier called by one warpgroup per PE (reference nvshmemx_barrier_warpgroup, its fourth thread
 * group scope: four warps that meet at a named hardware barrier, threadgroup/
 * nvshmemi_common_device_defines.cuh:76-110).  gfx950 has no barrier for part of a work-group, so the
 * wavefronts of the warpgroup - threads [256 g, 256 g + 256) of the block - meet at two words of
 * the team's sync row instead, an arrival count and a generation: every wavefront reads the
 * generation and adds one to the count; the last one to arrive puts the count back to zero and
 * advances the generation, the others wait for the generation to change.  The count is zero between
 * meetings, so groups of different sizes (a short last group) can follow each other.  The
 * warpgroup's first thread then runs the thread-scope barrier among the PEs, and a second meeting
 * releases the others.  As with the warp scope, only one warpgroup per PE may be inside a barrier
 * on a given team at a time. */
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_warpgroup_meet(nvshmem_team_t team) {
    const unsigned tid = nvshmemi_amd_block_tid(), nthr = nvshmemi_amd_block_size();
    const unsigned first = tid & ~(unsigned)(NVSHMEMI_AMD_WARPGROUP_SIZE - 1);
    const unsigned members = nthr - first < NVSHMEMI_AMD_WARPGROUP_SIZE ? nthr - first : NVSHMEMI_AMD_WARPGROUP_SIZE;
    const uint64_t waves = (members + NVSHMEMI_WARP_SIZE - 1) / NVSHMEMI_WARP_SIZE;
    uint64_t *count = nvshmemi_device_state_d.team_sync +
                      ((size_t)team * NVSHMEMI_AMD_MAX_PES + (size_t)nvshmemi_amd_my_pe()) * NVSHMEMI_AMD_TEAM_SYNC_WORDS +
                      NVSHMEMI_AMD_WARPGROUP_ARRIVE_WORD;
    uint64_t *generation = count + 1;
    const uint64_t seen = __hip_atomic_load(generation, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    /* the generation is read, and this wavefront's earlier memory operations are done, before it
     * reports its arrival */
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    if ((tid & (NVSHMEMI_WARP_SIZE - 1)) == 0) {
        if (__hip_atomic_fetch_add(count, (uint64_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == waves) {
            __hip_atomic_store(count, (uint64_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            /* release: the count is back at zero before anyone sees the new generation */
            __hip_atomic_store(generation, seen + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            nvshmemi_wait_until<uint64_t>(generation, NVSHMEM_CMP_NE, seen);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}
NVSHMEMI_DEVICE_INLINE int nvshmemi_barrier_warpgroup(nvshmem_team_t team) {
    if (nvshmemi_amd_team_view(team).size <= 0) return 1; /* the calling PE is not a member */
    nvshmemi_amd_warpgroup_meet(team);
    if ((nvshmemi_amd_block_tid() & (NVSHMEMI_AMD_WARPGROUP_SIZE - 1)) == 0)
        nvshmemi_barrier_threadgroup<NVSHMEMI_THREADGROUP_THREAD>(team);
    nvshmemi_amd_warpgroup_meet(team);
    return 0;
}

/* ------------------------------------------------------------------------------------------------
 * Reduction operator (reference perform_gpu_rdxn, coll/reduce.cuh:49-105): computed in the element
 * type; 16-bit floats add/multiply in fp32 and round to nearest-even once per step, which equals
 * the correctly rounded 16-bit operation.  min/max keep the reference's operand rule
 * `(a < b) ? a : b` / `(a > b) ? a : b`, which fixes the result for NaN and signed zeros.
 * Signed integer sum/prod wrap (computed unsigned).
 * ---------------------------------------------------------------------------------------------- */
template <typename T> struct nvshmemi_amd_arith { typedef T type; };
template <> struct nvshmemi_amd_arith<__hip_bfloat16> { typedef float type; };
template <> struct nvshmemi_amd_arith<__half> { typedef float type; };
template <> struct nvshmemi_amd_arith<signed char> { typedef unsigned char type; };
template <> struct nvshmemi_amd_arith<char> { typedef unsigned char type; };
template <> struct nvshmemi_amd_arith<short> { typedef unsigned short type; };
template <> struct nvshmemi_amd_arith<int> { typedef unsigned int type; };
template <> struct nvshmemi_amd_arith<long> { typedef unsigned long type; };
template <> struct nvshmemi_amd_arith<long long> { typedef unsigned long long type; };

template <typename T> NVSHMEMI_DEVICE_INLINE float nvshmemi_amd_to_float(T v) { return (float)v; }
template <> NVSHMEMI_DEVICE_INLINE float nvshmemi_amd_to_float(__hip_bfloat16 v) { return __bfloat162float(v); }
template <> NVSHMEMI_DEVICE_INLINE float nvshmemi_amd_to_float(__half v) { return __half2float(v); }
template <typename T> NVSHMEMI_DEVICE_INLINE T nvshmemi_amd_from_float(float v) { return (T)v; }
template <> NVSHMEMI_DEVICE_INLINE __hip_bfloat16 nvshmemi_amd_from_float(float v) { return __float2bfloat16(v); }
template <> NVSHMEMI_DEVICE_INLINE __half nvshmemi_amd_from_float(float v) { return __float2half_rn(v); }

template <typename T> struct nvshmemi_amd_is_half { static constexpr bool value = false; };
template <> struct nvshmemi_amd_is_half<__hip_bfloat16> { static constexpr bool value = true; };
template <> struct nvshmemi_amd_is_half<__half> { static constexpr bool value = true; };

template <typename T, int OP>
NVSHMEMI_DEVICE_INLINE T nvshmemi_amd_reduce_op(T a, T b) {
    typedef typename nvshmemi_amd_arith<T>::type A;
    if constexpr (nvshmemi_amd_is_half<T>::value) {
        const float fa = nvshmemi_amd_to_float(a), fb = nvshmemi_amd_to_float(b);
        if constexpr (OP == NVSHMEMI_OP_sum) return nvshmemi_amd_from_float<T>(fa + fb);
        if constexpr (OP == NVSHMEMI_OP_prod) return nvshmemi_amd_from_float<T>(fa * fb);
        if constexpr (OP == NVSHMEMI_OP_min) return (fa < fb) ? a : b;
        if constexpr (OP == NVSHMEMI_OP_max) return (fa > fb) ? a : b;
        return a;
    } else {
        if constexpr (OP == NVSHMEMI_OP_sum) return (T)((A)a + (A)b);
        if constexpr (OP == NVSHMEMI_OP_prod) return (T)((A)a * (A)b);
        if constexpr (OP == NVSHMEMI_OP_min) return (a < b) ? a : b;
        if constexpr (OP == NVSHMEMI_OP_max) return (a > b) ? a : b;
        if constexpr (std::is_integral<T>::value) {
            if constexpr (OP == NVSHMEMI_OP_and) return (T)(a & b);
            if constexpr (OP == NVSHMEMI_OP_or) return (T)(a | b);
            if constexpr (OP == NVSHMEMI_OP_xor) return (T)(a ^ b);
        }
        return a;
    }
}

/* Fold of one element over the PEs in the fixed order of the reference's gather-then-fold path
 * (coll/reduce.cuh:1297-1303): acc = op(x0, x1); acc = op(x_i, acc) for i = 2..n-1. */
template <typename T, int OP>
NVSHMEMI_DEVICE_INLINE T nvshmemi_amd_fold_step(int i, T acc, T x) {
    return (i == 1) ? nvshmemi_amd_reduce_op<T, OP>(acc, x) : nvshmemi_amd_reduce_op<T, OP>(x, acc);
}

/* The form an accumulator takes between the steps of a fold.  For most types it is the element itself.  A
 * bf16 sum or product keeps it as the fp32 value of the rounded bf16 (the bf16's bits in the high half of the
 * word), which v_cvt_pk_bf16_f32 writes directly when the value is its second operand: a step is then
 * add + convert instead of add + convert + shift, with the same rounding, once per step. */
template <typename T, int OP>
struct nvshmemi_amd_fold_form {
    typedef T acc_t;
    static NVSHMEMI_DEVICE_INLINE acc_t lift(T x) { return x; }
    static NVSHMEMI_DEVICE_INLINE acc_t step(int i, acc_t acc, T x) { return nvshmemi_amd_fold_step<T, OP>(i, acc, x); }
    static NVSHMEMI_DEVICE_INLINE T lower(acc_t acc) { return acc; }
};
template <int OP>
struct nvshmemi_amd_bf16_float_form {
    typedef float acc_t;
    static NVSHMEMI_DEVICE_INLINE acc_t lift(__hip_bfloat16 x) {
        return __builtin_bit_cast(float, (unsigned)__builtin_bit_cast(unsigned short, x) << 16);
    }
    static NVSHMEMI_DEVICE_INLINE acc_t step(int i, acc_t acc, __hip_bfloat16 x) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        typedef float floatx2 __attribute__((ext_vector_type(2)));
        const float a = (i == 1) ? acc : lift(x), b = (i == 1) ? lift(x) : acc;
        const floatx2 wide = {0.0f, OP == NVSHMEMI_OP_sum ? a + b : a * b};
        return __builtin_bit_cast(float, __builtin_convertvector(wide, bf16x2));
    }
    static NVSHMEMI_DEVICE_INLINE __hip_bfloat16 lower(acc_t acc) {
        return __builtin_bit_cast(__hip_bfloat16, (unsigned short)(__builtin_bit_cast(unsigned, acc) >> 16));
    }
};
template <> struct nvshmemi_amd_fold_form<__hip_bfloat16, NVSHMEMI_OP_sum> : nvshmemi_amd_bf16_float_form<NVSHMEMI_OP_sum> {};
template <> struct nvshmemi_amd_fold_form<__hip_bfloat16, NVSHMEMI_OP_prod> : nvshmemi_amd_bf16_float_form<NVSHMEMI_OP_prod> {};

/* ------------------------------------------------------------------------------------------------
 * Low-latency packets for small collectives (the role of the reference's LL protocol,
 * non_abi/device/common/nvshmemi_common_device.cuh:981-1066 packLL / recvLL, used by
 * coll/fcollect.cuh:100-314 and coll/broadcast.cuh:40-273).
 *
 * Eight payload bytes travel as one 16-byte packet {lo32, flag, hi32, flag}: each 8-byte half
 * carries its own copy of the flag, so a receiver that sees the expected flag in a half also sees
 * that half's data.  No fence and no barrier is needed: packets are written and polled with
 * agent-scope (write-through / L2-bypassing) accesses.  The flag is the team's call counter (never
 * 0, buffers start zeroed), and consecutive calls rotate through three buffers.  Call f overwrites
 * the buffer of call f-3, so every member must have finished reading f-3 by then.  A PE that
 * completed an fcollect or reduce f-1 has received packets of f-1 from every member, each of which
 * had finished reading f-2 before it sent them.  A broadcast gives its root no such knowledge, so a
 * root waits until every receiver has published `done >= f-2`; a receiver that then completes the
 * broadcast f-1 inherits "everybody finished f-3".
 *
 * An agent-scope access costs about a memory round trip per instruction, whether one lane is active
 * or 64, so the packets of a call are spread over the lanes - one per lane - and the path is only
 * taken while that is possible; longer messages are faster through the copy engine and a barrier.
 * The choice depends on the message size and on the size of the calling thread group, so all
 * members of a team must make a collective call with the same scope and group size (they do when
 * one launch carries all PEs).  The 32-bit flags and `done` counters are compared as plain
 * integers: the protocol assumes fewer than 2^32 packet calls per team handle life.
 * ---------------------------------------------------------------------------------------------- */
NVSHMEMI_DEVICE_INLINE char *nvshmemi_amd_ll_buffer(nvshmem_team_t team, int pe, uint32_t flag) {
    const size_t buf = 2 * (size_t)NVSHMEMI_AMD_LL_PAYLOAD_BYTES;
    return nvshmemi_device_state_d.ll_buffers +
           (((size_t)team * (size_t)nvshmemi_device_state_d.npes + (size_t)pe) * NVSHMEMI_AMD_LL_BUFFERS +
            flag % NVSHMEMI_AMD_LL_BUFFERS) * buf;
}
NVSHMEMI_DEVICE_INLINE uint64_t *nvshmemi_amd_ll_word(nvshmem_team_t team, int pe, int word) {
    return nvshmemi_device_state_d.team_sync +
           ((size_t)team * NVSHMEMI_AMD_MAX_PES + (size_t)pe) * NVSHMEMI_AMD_TEAM_SYNC_WORDS + word;
}
NVSHMEMI_DEVICE_INLINE unsigned nvshmemi_amd_ll_packets(size_t nbytes) { return (unsigned)((nbytes + 7) >> 3); }

/* Packets one call may receive per PE: one per lane of the thread group; a single thread takes a
 * few, one after the other, which still beats its barrier. */
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE unsigned nvshmemi_amd_ll_lanes() {
    const unsigned nthr = (unsigned)nvshmemi_threadgroup_size<SCOPE>();
    return nthr < 8 ? 8 : nthr;
}
NVSHMEMI_DEVICE_INLINE bool nvshmemi_amd_ll_available() { return nvshmemi_device_state_d.ll_buffers != nullptr; }

/* The calling PE's count of packet collectives on `team` so far.  Every thread of the group reads
 * it; no group synchronisation is needed in front: the word only changes in nvshmemi_amd_ll_next_flag,
 * and every packet collective passes nvshmemi_amd_ll_publish_done's synchronisation after that. */
NVSHMEMI_DEVICE_INLINE uint64_t nvshmemi_amd_ll_peek_count(nvshmem_team_t team) {
    return *reinterpret_cast<volatile uint64_t *>(
        nvshmemi_amd_ll_word(team, nvshmemi_amd_my_pe(), NVSHMEMI_AMD_LL_COUNT_WORD));
}
/* Next flag of the calling PE for `team`, from the count peeked earlier; all threads of the group
 * return the same value.  The synchronisation keeps the first thread's update behind everybody's read. */
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE uint32_t nvshmemi_amd_ll_next_flag(nvshmem_team_t team, uint64_t count_seen) {
    uint32_t flag = (uint32_t)count_seen + 1u;
    if (flag == 0) flag = 1; /* 0 is what an empty buffer holds */
    nvshmemi_threadgroup_sync<SCOPE>();
    if (nvshmemi_thread_id_in_threadgroup<SCOPE>() == 0)
        *reinterpret_cast<volatile uint64_t *>(
            nvshmemi_amd_ll_word(team, nvshmemi_amd_my_pe(), NVSHMEMI_AMD_LL_COUNT_WORD)) = flag;
    return flag;
}
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE uint32_t nvshmemi_amd_ll_next_flag(nvshmem_team_t team) {
    return nvshmemi_amd_ll_next_flag<SCOPE>(team, nvshmemi_amd_ll_peek_count(team));
}

NVSHMEMI_DEVICE_INLINE uint64_t nvshmemi_amd_ll_load_payload(const char *src, size_t left) {
    uint64_t w = 0;
    if (left >= 8 && (((uintptr_t)src) & 7) == 0) return *reinterpret_cast<const uint64_t *>(src);
    const size_t n = left < 8 ? left : 8;
    for (size_t b = 0; b < n; ++b) w |= (uint64_t)(unsigned char)src[b] << (8 * b);
    return w;
}
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_ll_store_payload(char *dst, uint64_t w, size_t left) {
    if (left >= 8 && (((uintptr_t)dst) & 7) == 0) {
        *reinterpret_cast<uint64_t *>(dst) = w;
        return;
    }
    const size_t n = left < 8 ? left : 8;
    for (size_t b = 0; b < n; ++b) dst[b] = (char)(w >> (8 * b));
}
/* One packet, written with a single 16-byte agent-scope store so that a wavefront's packets fill
 * whole cache lines; only the two 8-byte halves have to arrive untorn. */
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_ll_store_packet(char *packet, uint64_t w, uint32_t flag) {
    nvshmemi_v4u v;
    v.x = (uint32_t)w;
    v.y = flag;
    v.z = (uint32_t)(w >> 32);
    v.w = flag;
    nvshmemi_amd_store16_agent(packet, v);
}
/* Waits until both halves of the packet carry `flag` and returns its 8 payload bytes.  A bounded
 * wait that gives up records the timeout like nvshmemi_wait_until and returns what it last saw. */
NVSHMEMI_DEVICE_INLINE uint64_t nvshmemi_amd_ll_recv_packet(const char *packet, uint32_t flag) {
    const uint64_t limit = nvshmemi_device_state_d.spin_limit;
    uint64_t polls = 0;
    nvshmemi_v4u v;
    for (;;) {
        asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(packet) : "memory");
        if (v.y == flag && v.w == flag) break;
        if (limit && ++polls > limit) {
            nvshmemi_amd_record_timeout(packet, v.y, flag);
            break;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    return (uint64_t)v.x | ((uint64_t)v.z << 32);
}
/* Sends npk chunks to each other member of the team, chunk j into slot slot0 + j of its buffers:
 * the chunks of src for everybody (dest_stride 0), or those of src + idx * dest_stride for member
 * idx.  The (member, chunk) pairs are spread over the lanes. */
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_ll_send_to_all(nvshmem_team_t team, const nvshmemi_amd_team_view_t &tv,
                                                        const char *src, size_t nbytes, unsigned npk,
                                                        unsigned slot0, uint32_t flag, size_t dest_stride = 0) {
    if (SCOPE == NVSHMEMI_THREADGROUP_THREAD) {
        /* a single thread: chunk by chunk, the chunk loaded once (dest_stride 0) or for eight members in
         * one go, then the stores to the members one behind the other with no load in between (member
         * by member every store waited for the load in front of it: 8 bytes among 8 PEs, fcollect 7.0 us
         * against 5.2 us, allreduce 5.9 against 3.6) */
        for (unsigned j = 0; j < npk; ++j) {
            const uint64_t same =
                dest_stride ? 0 : nvshmemi_amd_ll_load_payload(src + 8 * (size_t)j, nbytes - 8 * (size_t)j);
            for (int o0 = 0; o0 < tv.size - 1; o0 += 8) {
                uint64_t x[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int off = o0 + k < tv.size - 1 ? o0 + k : o0;
                    int idx = tv.my_pe + 1 + off;
                    if (idx >= tv.size) idx -= tv.size;
                    x[k] = dest_stride ? nvshmemi_amd_ll_load_payload(src + (size_t)idx * dest_stride + 8 * (size_t)j,
                                                                      nbytes - 8 * (size_t)j)
                                       : same;
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    if (o0 + k >= tv.size - 1) break;
                    int idx = tv.my_pe + 1 + o0 + k;
                    if (idx >= tv.size) idx -= tv.size;
                    nvshmemi_amd_ll_store_packet(
                        nvshmemi_amd_ll_buffer(team, nvshmemi_amd_team_pe(tv, idx), flag) + (size_t)(slot0 + j) * 16, x[k],
                        flag);
                }
            }
        }
        return;
    }
    const unsigned nthr = (unsigned)nvshmemi_threadgroup_size<SCOPE>();
    const unsigned total = (unsigned)(tv.size - 1) * npk;
    for (unsigned w = (unsigned)nvshmemi_thread_id_in_threadgroup<SCOPE>(); w < total; w += nthr) {
        const unsigned off = w / npk, j = w - off * npk;
        int idx = tv.my_pe + 1 + (int)off;
        if (idx >= tv.size) idx -= tv.size;
        nvshmemi_amd_ll_store_packet(
            nvshmemi_amd_ll_buffer(team, nvshmemi_amd_team_pe(tv, idx), flag) + (size_t)(slot0 + j) * 16,
            nvshmemi_amd_ll_load_payload(src + (size_t)idx * dest_stride + 8 * (size_t)j, nbytes - 8 * (size_t)j),
            flag);
    }
}
/* Tells the other PEs that this PE has read everything of call `flag`. */
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_ll_publish_done(nvshmem_team_t team, uint32_t flag) {
    nvshmemi_threadgroup_sync<SCOPE>();
    if (nvshmemi_thread_id_in_threadgroup<SCOPE>() == 0)
        __hip_atomic_store(nvshmemi_amd_ll_word(team, nvshmemi_amd_my_pe(), NVSHMEMI_AMD_LL_DONE_WORD),
                           (uint64_t)flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
/* fcollect / reduce: a contribution of nbytes from each of `size` members */
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE bool nvshmemi_amd_ll_fits(size_t nbytes, int size) {
    const size_t npk = (nbytes + 7) >> 3;
    return nbytes > 0 && nbytes <= NVSHMEMI_AMD_LL_MAX_BYTES && nvshmemi_amd_ll_available() &&
           npk * 8 * (size_t)size <= NVSHMEMI_AMD_LL_PAYLOAD_BYTES &&
           npk * (size_t)(size - 1) <= nvshmemi_amd_ll_lanes<SCOPE>();
}

/* Small allreduce in one hop: every member sends its source to every other member as packets and
 * folds the contributions itself, in member order.  Wavefront and block scope: lane (chunk j,
 * member p) fetches one packet (its own source for p == me), then the lanes of a chunk - adjacent,
 * in a group of G = npes rounded up to a power of two - pass their values to each other with
 * cross-lane reads and the first lane of the group stores the result. */
template <typename T, int OP, int SCOPE, bool SCATTER = false>
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_ll_reduce(nvshmem_team_t team, const nvshmemi_amd_team_view_t &tv,
                                                   T *dest, const T *source, size_t nreduce, unsigned group) {
    constexpr size_t PER = 8 / sizeof(T);
    const int me = tv.my_pe, npes = tv.size;
    const unsigned tid = (unsigned)nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const size_t nbytes = nreduce * sizeof(T);
    const uint32_t flag = nvshmemi_amd_ll_next_flag<SCOPE>(team);
    const unsigned npk = nvshmemi_amd_ll_packets(nbytes);
    /* reducescatter (SCATTER): member idx is sent block idx of the source and folds the blocks
     * `me` it receives, with the operands in reducescatter's order */
    const char *src_all = nvshmemi_amd_local(source);
    const char *src = src_all + (SCATTER ? (size_t)me * nbytes : 0);
    char *dst = nvshmemi_amd_local(dest);
    nvshmemi_amd_ll_send_to_all<SCOPE>(team, tv, src_all, nbytes, npk, (unsigned)me * npk, flag,
                                       SCATTER ? nbytes : 0);
    /* dest may be source: everything is sent before any result is stored */
    nvshmemi_threadgroup_sync<SCOPE>();
    const char *mine = nvshmemi_amd_ll_buffer(team, nvshmemi_amd_my_pe(), flag);
    if (SCOPE == NVSHMEMI_THREADGROUP_THREAD) {
        for (unsigned j = 0; j < npk; ++j) {
            T acc[PER];
            for (int p = 0; p < npes; ++p) {
                const uint64_t v = p == me ? nvshmemi_amd_ll_load_payload(src + 8 * (size_t)j, nbytes - 8 * (size_t)j)
                                           : nvshmemi_amd_ll_recv_packet(mine + ((size_t)p * npk + j) * 16, flag);
                T x[PER];
                __builtin_memcpy(x, &v, 8);
#pragma unroll
                for (size_t k = 0; k < PER; ++k)
                    acc[k] = p == 0 ? x[k]
                                    : SCATTER ? nvshmemi_amd_reduce_op<T, OP>(acc[k], x[k])
                                              : nvshmemi_amd_fold_step<T, OP>(p, acc[k], x[k]);
            }
            uint64_t r;
            __builtin_memcpy(&r, acc, 8);
            nvshmemi_amd_ll_store_payload(dst + 8 * (size_t)j, r, nbytes - 8 * (size_t)j);
        }
    } else {
        /* group * npk <= nthr: every (chunk, member) pair has a lane; whole wavefronts take part in
         * the cross-lane reads, lanes without a pair carry zeros */
        const unsigned gshift = 31u - (unsigned)__builtin_clz(group);
        const unsigned j = tid >> gshift, p = tid & (group - 1);
        const bool wave_active = (tid & ~63u) < group * npk;
        if (wave_active) {
            uint64_t v = 0;
            if (j < npk && (int)p < npes)
                v = (int)p == me ? nvshmemi_amd_ll_load_payload(src + 8 * (size_t)j, nbytes - 8 * (size_t)j)
                                 : nvshmemi_amd_ll_recv_packet(mine + ((size_t)p * npk + j) * 16, flag);
            const int base = (int)((tid & 63u) & ~(group - 1));
            T acc[PER];
            for (int q = 0; q < npes; ++q) {
                const uint64_t xv = (uint64_t)__shfl((unsigned long long)v, base + q, 64);
                T x[PER];
                __builtin_memcpy(x, &xv, 8);
#pragma unroll
                for (size_t k = 0; k < PER; ++k)
                    acc[k] = q == 0 ? x[k]
                                    : SCATTER ? nvshmemi_amd_reduce_op<T, OP>(acc[k], x[k])
                                              : nvshmemi_amd_fold_step<T, OP>(q, acc[k], x[k]);
            }
            if (p == 0 && j < npk) {
                uint64_t r;
                __builtin_memcpy(&r, acc, 8);
                nvshmemi_amd_ll_store_payload(dst + 8 * (size_t)j, r, nbytes - 8 * (size_t)j);
            }
        }
    }
    nvshmemi_amd_ll_publish_done<SCOPE>(team, flag);
}
/* the group width of nvshmemi_amd_ll_reduce, or 0 when the call does not qualify */
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE unsigned nvshmemi_amd_ll_reduce_group(size_t nbytes, int size) {
    if (!nvshmemi_amd_ll_fits<SCOPE>(nbytes, size)) return 0;
    if (SCOPE == NVSHMEMI_THREADGROUP_THREAD) return 1;
    unsigned group = 1;
    while ((int)group < size) group <<= 1;
    return group * (unsigned)((nbytes + 7) >> 3) <= (unsigned)nvshmemi_threadgroup_size<SCOPE>() ? group : 0;
}

/* ------------------------------------------------------------------------------------------------
 * Line packets: the reference's LL128 (128-byte lines with one flag word,
 * non_abi/device/common/nvshmemi_common_device.cuh:699-920, used by coll/fcollect.cuh:157-314)
 * re-derived for this GPU.
 *
 * The unit is HALF a cache line: 64 bytes = 56 bytes of payload and an 8-byte flag word, written by
 * four adjacent lanes with one 16-byte agent-scope store each - lane k of the four carries payload
 * bytes [16 k, 16 k + 16), the last lane 8 bytes and the flag.  The compute unit sends a wavefront's
 * stores to the L2 as 64-byte requests and the L2 writes them through as 64-byte requests, so a unit
 * travels as one write and a receiver that finds the flag finds the payload (the protocol assumes
 * that such a write is not torn; tests stream changing data through it and check every unit).  A
 * 128-byte line with ONE flag would need the two requests of a line to arrive together, which nothing
 * promises here.  56 bytes are a whole number of elements of every type, so a lane folds whole
 * elements.  Efficiency 7/8 against the 1/2 of the 16-byte packets, and a block of 256 threads covers
 * 3.5 KiB per member with one unit-lane per thread.
 *
 * Allreduce / reducescatter in one hop, no barrier: thread (u, k) - unit u, lane k - sends its 16
 * bytes of the PE's contribution to every other member's buffer (slot `me`), then fetches the same
 * position of every member's slot in its own buffer, all loads issued before the first check; the
 * wavefront repeats the batch until every unit it covers carries the call's flag, and the lane folds
 * its elements in member order and stores them.  Flags, buffer rotation and the `done` word are those
 * of the 16-byte packets above (the two formats share the buffers: a stale word of the other format
 * cannot equal a later call's flag word).
 *
 * Compiled in only where the including translation unit defines NVSHMEMI_AMD_UNIT_PACKETS (every
 * member's code must then be built that way).  It measured no faster than the staged one-barrier form
 * it would replace (8 PEs, 256 threads: 1 KiB per member 3.83 against 3.41 us, 2 KiB 3.84 against
 * 3.80), and its mere presence in a kernel - as a branch never taken - cost the reducescatter beside
 * it 1.2 us per call, so the default build leaves it out.
 * ---------------------------------------------------------------------------------------------- */
#define NVSHMEMI_AMD_UNIT_BYTES 64
#define NVSHMEMI_AMD_UNIT_PAYLOAD 56
NVSHMEMI_DEVICE_INLINE unsigned nvshmemi_amd_units(size_t nbytes) {
    return (unsigned)((nbytes + NVSHMEMI_AMD_UNIT_PAYLOAD - 1) / NVSHMEMI_AMD_UNIT_PAYLOAD);
}
/* one unit-lane per thread, all members' slots in one buffer, buffers at hand */
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE bool nvshmemi_amd_units_fit(size_t nbytes, int npes) {
    const size_t units = (nbytes + NVSHMEMI_AMD_UNIT_PAYLOAD - 1) / NVSHMEMI_AMD_UNIT_PAYLOAD;
    const size_t nthr = (size_t)nvshmemi_threadgroup_size<SCOPE>();
    return SCOPE != NVSHMEMI_THREADGROUP_THREAD && nbytes > 0 && nvshmemi_amd_ll_available() && (nthr & 3) == 0 &&
           4 * units <= nthr && (size_t)npes * units * NVSHMEMI_AMD_UNIT_BYTES <= 2 * (size_t)NVSHMEMI_AMD_LL_PAYLOAD_BYTES;
}
/* the 16 bytes lane k of unit u carries: payload from src (zeros behind its end), for k == 3 the flag word on top */
NVSHMEMI_DEVICE_INLINE nvshmemi_v4u nvshmemi_amd_unit_pack(const char *src, size_t nbytes, unsigned u, unsigned k,
                                                           uint32_t flag) {
    const size_t at = (size_t)u * NVSHMEMI_AMD_UNIT_PAYLOAD + 16 * k;
    const size_t want = k == 3 ? 8 : 16;
    nvshmemi_v4u x = {0, 0, 0, 0};
    if (at + want <= nbytes) {
        if (k == 3) {
            uint64_t w;
            __builtin_memcpy(&w, src + at, 8);
            x.x = (uint32_t)w;
            x.y = (uint32_t)(w >> 32);
        } else {
            x = nvshmemi_amd_load16<false>(src + at);
        }
    } else if (at < nbytes) {
        unsigned char b[16] = {0};
        for (size_t i = 0; at + i < nbytes && i < want; ++i) b[i] = (unsigned char)src[at + i];
        __builtin_memcpy(&x, b, 16);
    }
    if (k == 3) {
        x.z = flag;
        x.w = flag;
    }
    return x;
}
template <typename T, int OP, int SCOPE, bool SCATTER>
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_unit_reduce(nvshmem_team_t team, const nvshmemi_amd_team_view_t &tv, T *dest,
                                                     const T *source, size_t nreduce) {
    constexpr size_t VEC = 16 / sizeof(T);
    union pack_t {
        nvshmemi_v4u v;
        T e[VEC];
    };
    const int me = tv.my_pe, npes = tv.size;
    const unsigned tid = (unsigned)nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const size_t nbytes = nreduce * sizeof(T);
    const unsigned units = nvshmemi_amd_units(nbytes);
    const unsigned u = tid >> 2, k = tid & 3;
    const bool active = u < units;
    const uint32_t flag = nvshmemi_amd_ll_next_flag<SCOPE>(team);
    const char *src_all = nvshmemi_amd_local(source);
    /* SCATTER: member idx is sent block idx of the source and folds the blocks `me` it receives */
    const size_t slot_off = ((size_t)me * units + u) * NVSHMEMI_AMD_UNIT_BYTES + 16 * k;
    if (active) {
        const nvshmemi_v4u same = SCATTER ? nvshmemi_v4u{0, 0, 0, 0} : nvshmemi_amd_unit_pack(src_all, nbytes, u, k, flag);
        for (int off = 1; off < npes; ++off) {
            const int idx = me + off < npes ? me + off : me + off - npes;
            const nvshmemi_v4u x = SCATTER ? nvshmemi_amd_unit_pack(src_all + (size_t)idx * nbytes, nbytes, u, k, flag) : same;
            nvshmemi_amd_store16_agent(nvshmemi_amd_ll_buffer(team, nvshmemi_amd_team_pe(tv, idx), flag) + slot_off, x);
        }
    }
    /* (dest may be source: a lane stores only the bytes whose source it has read itself) */
    const char *mine = nvshmemi_amd_ll_buffer(team, nvshmemi_amd_my_pe(), flag);
    const size_t at = (size_t)u * NVSHMEMI_AMD_UNIT_PAYLOAD + 16 * k;
    const uint64_t limit = nvshmemi_device_state_d.spin_limit;
    pack_t acc;
    acc.v = nvshmemi_v4u{0, 0, 0, 0};
    for (int p0 = 0; p0 < npes; p0 += 8) {
        pack_t x[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) x[q].v = nvshmemi_v4u{0, 0, 0, 0};
        uint64_t polls = 0;
        for (;;) {
            bool missing = false;
            /* The eight loads and their wait are ONE statement: between separate statements the compiler could
             * copy or spill a destination register while its load is still in flight.  A slot that has nothing
             * to fetch (an inactive lane, a member past the team, the PE itself) reads the start of the PE's own
             * buffer, which is always mapped, and its value is not used. */
            const char *from[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int p = p0 + q;
                from[q] = (active && p < npes && p != me)
                              ? mine + ((size_t)p * units + u) * NVSHMEMI_AMD_UNIT_BYTES + 16 * k
                              : mine;
            }
            asm volatile(
                "global_load_dwordx4 %0, %8, off sc1\n\t"
                "global_load_dwordx4 %1, %9, off sc1\n\t"
                "global_load_dwordx4 %2, %10, off sc1\n\t"
                "global_load_dwordx4 %3, %11, off sc1\n\t"
                "global_load_dwordx4 %4, %12, off sc1\n\t"
                "global_load_dwordx4 %5, %13, off sc1\n\t"
                "global_load_dwordx4 %6, %14, off sc1\n\t"
                "global_load_dwordx4 %7, %15, off sc1\n\t"
                "s_waitcnt vmcnt(0)"
                : "=&v"(x[0].v), "=&v"(x[1].v), "=&v"(x[2].v), "=&v"(x[3].v), "=&v"(x[4].v), "=&v"(x[5].v),
                  "=&v"(x[6].v), "=&v"(x[7].v)
                : "v"(from[0]), "v"(from[1]), "v"(from[2]), "v"(from[3]), "v"(from[4]), "v"(from[5]), "v"(from[6]),
                  "v"(from[7])
                : "memory");
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int p = p0 + q;
                if (active && k == 3 && p < npes && p != me) missing |= x[q].v.z != flag || x[q].v.w != flag;
            }
            if (!__builtin_amdgcn_ballot_w64(missing)) break;
            if (limit && ++polls > limit) {
                if (missing) nvshmemi_amd_record_timeout(mine, 0, flag);
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        if (active) {
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int p = p0 + q;
                if (p >= npes) break;
                if (p == me) x[q].v = nvshmemi_amd_unit_pack(src_all + (SCATTER ? (size_t)me * nbytes : 0), nbytes, u, k, flag);
                if (p == 0) {
                    acc = x[q];
                } else {
#pragma unroll
                    for (size_t e = 0; e < VEC; ++e)
                        acc.e[e] = SCATTER ? nvshmemi_amd_reduce_op<T, OP>(acc.e[e], x[q].e[e])
                                           : nvshmemi_amd_fold_step<T, OP>(p, acc.e[e], x[q].e[e]);
                }
            }
        }
    }
    if (active && at < nbytes) {
        char *dst = nvshmemi_amd_local(dest) + at;
        const size_t room = (k == 3 ? 8 : 16), left = nbytes - at < room ? nbytes - at : room;
        if (left == 16 && (((uintptr_t)dst) & 15) == 0) {
            *reinterpret_cast<nvshmemi_v4u *>(dst) = acc.v;
        } else {
            for (size_t e = 0; e * sizeof(T) < left; ++e) reinterpret_cast<T *>(dst)[e] = acc.e[e];
        }
    }
    nvshmemi_amd_ll_publish_done<SCOPE>(team, flag);
}

/* ------------------------------------------------------------------------------------------------
 * Collectives called from inside a user kernel, one thread group per PE
 * (reference coll/reduce.cuh:1158-1196 get-based reduce, coll/fcollect.cuh:331-344,
 * coll/alltoall.cuh:122-143).  Calls small enough for the packets above return when the caller's
 * own dest is complete; the others end with a barrier of the team.
 * ---------------------------------------------------------------------------------------------- */
/* One push to every member of the team in a single pass, for the all-push collectives below: member
 * idx receives the `nbytes` at src + idx * src_stride (src_stride 0: everybody receives the same
 * bytes) at the symmetric address dst_sym.  A lane loads each of its vectors once - for different
 * sources, from all of them before the first store - and stores it to every member, in the
 * reference's order me, me + 1, ...; a loop of whole copies, one member after the other, pays the load
 * latency once per member instead (fcollect of 2 KiB per member among 8 PEs with 256 threads,
 * barrier included: 2.8 us against 4.9 us).  Needs a wavefront or block, source and destination on
 * the same offset within 16 bytes and a stride that keeps it; returns false, having done nothing,
 * otherwise, and for different sources longer than NVSHMEMI_AMD_FANOUT_MAX_BYTES each, where a copy
 * per member with the copy engine's longer rounds is as fast or faster (one source for all stays ahead
 * at every size: 64 KiB per member among 8 PEs with 256 threads 8.6 against 12.9 us, 1 MiB 98 against
 * 131 us). */
#define NVSHMEMI_AMD_FANOUT_MAX_BYTES 32768
/* in-kernel broadcasts from this size on are fetched by every PE instead of pushed by the root */
#define NVSHMEMI_AMD_BCAST_PULL_BYTES 32768
#define NVSHMEMI_AMD_BCAST_PULL_BYTES_PER_LANE 128
/* (every PE's slice starts on a multiple of 16 bytes and more, so a symmetric address and its
 * translations share their low bits and every PE decides alike) */
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE bool nvshmemi_amd_fanout_fits(const void *dst, const void *src, size_t src_stride,
                                                     size_t nbytes) {
    return SCOPE != NVSHMEMI_THREADGROUP_THREAD && (src_stride == 0 || nbytes <= NVSHMEMI_AMD_FANOUT_MAX_BYTES) &&
           (src_stride & 15) == 0 && ((((uintptr_t)dst) ^ (uintptr_t)src) & 15) == 0;
}
template <int SCOPE>
NVSHMEMI_DEVICE_INLINE bool nvshmemi_amd_fanout_copy(const nvshmemi_amd_team_view_t &tv, void *dst_sym,
                                                     const char *src, size_t src_stride, size_t nbytes) {
    if (!nvshmemi_amd_fanout_fits<SCOPE>(dst_sym, src, src_stride, nbytes)) return false;
    const int me = tv.my_pe, npes = tv.size;
    const size_t tid = (size_t)nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const size_t nthr = (size_t)nvshmemi_threadgroup_size<SCOPE>();
    size_t head = (size_t)(-(uintptr_t)src & 15);
    if (head > nbytes) head = nbytes;
    const size_t nvec = (nbytes - head) / 16;
    const size_t body_end = head + 16 * nvec;
    /* the bytes in front of the first and behind the last whole vector */
    for (size_t b = tid; b < head + (nbytes - body_end); b += nthr) {
        const size_t pos = b < head ? b : body_end + (b - head);
        for (int ii = 0; ii < npes; ++ii) {
            const int idx = me + ii < npes ? me + ii : me + ii - npes;
            nvshmemi_amd_remote(dst_sym, nvshmemi_amd_team_pe(tv, idx))[pos] = src[(size_t)idx * src_stride + pos];
        }
    }
    for (size_t v = tid; v < nvec; v += nthr) {
        const size_t pos = head + 16 * v;
        if (src_stride == 0) {
            const nvshmemi_v4u x = nvshmemi_amd_load16<true>(src + pos);
            for (int ii = 0; ii < npes; ++ii) {
                const int idx = me + ii < npes ? me + ii : me + ii - npes;
                nvshmemi_amd_stream_store16(nvshmemi_amd_remote(dst_sym, nvshmemi_amd_team_pe(tv, idx)) + pos, x);
            }
        } else {
            for (int i0 = 0; i0 < npes; i0 += 8) {
                nvshmemi_v4u x[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int ii = i0 + k < npes ? i0 + k : npes - 1; /* past the end: the last member once more */
                    const int idx = me + ii < npes ? me + ii : me + ii - npes;
                    x[k] = nvshmemi_amd_load16<true>(src + (size_t)idx * src_stride + pos);
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int ii = i0 + k < npes ? i0 + k : npes - 1;
                    const int idx = me + ii < npes ? me + ii : me + ii - npes;
                    nvshmemi_amd_stream_store16(nvshmemi_amd_remote(dst_sym, nvshmemi_amd_team_pe(tv, idx)) + pos, x[k]);
                }
            }
        }
    }
    return true;
}

/* Reduce: PE `me` owns the element range [me*chunk, (me+1)*chunk): it folds that range from every
 * PE's source and stores the result into every PE's dest.  Each element is read by exactly one lane
 * before that lane overwrites it, so source == dest is safe, and every source byte is read once.
 * When both buffers are 16-byte aligned the range is cut on vector boundaries and moved as
 * dwordx4; otherwise element by element. */
template <typename T, int OP>
NVSHMEMI_DEVICE_INLINE T nvshmemi_amd_fold_element(const T *src0, size_t pe_stride, int npes, size_t i) {
    T acc = src0[i];
    for (int pe = 1; pe < npes; ++pe)
        acc = nvshmemi_amd_fold_step<T, OP>(pe, acc, src0[(size_t)pe * pe_stride + i]);
    return acc;
}

/* Reductions of a few KiB in one hop and ONE barrier: every member pushes its whole contribution
 * (SCATTER: block idx of it to member idx) into slot `me` of every member's staging buffer, a lane
 * storing each vector it loaded to all members; after the barrier every PE folds the slots of its own
 * buffer in member order - all slots' vectors fetched before the first fold - and writes only its own
 * dest.  The gather form below needs a barrier on either side.  The team's count of synchronisations
 * picks one of two buffers by its parity: a member that pushes into a buffer again has passed a later
 * synchronisation, which every member entered only after it had folded the earlier contents.
 * Needs a wavefront or block, source and dest on multiples of 16 bytes (symmetric addresses, so
 * every PE decides alike), for SCATTER blocks of whole vectors, and all slots in one buffer. */
template <int SCOPE, bool SCATTER>
NVSHMEMI_DEVICE_INLINE bool nvshmemi_amd_staged_fits(const void *dest, const void *source, size_t nbytes, int npes) {
    const size_t slot = (nbytes + 15) & ~(size_t)15;
    /* what one PE pushes and reads back grows with npes * nbytes, and beyond 8 (SCATTER: 4, and 16 KiB in
     * all) vectors per lane the gather form with its two barriers is the faster one again (8 PEs, 256
     * threads, fp32 sum: 3.5 against 4.9 us at 512 B and 1 KiB per member, 3.8 at 2 KiB, 4.5 at 4 KiB) */
    const size_t per_lane = SCATTER ? 64 : 128;
    return SCOPE != NVSHMEMI_THREADGROUP_THREAD && nvshmemi_amd_ll_available() && nbytes > 0 &&
           (size_t)npes * slot <= (SCATTER ? NVSHMEMI_AMD_STAGE_BYTES / 2 : NVSHMEMI_AMD_STAGE_BYTES) &&
           (size_t)npes * slot <= per_lane * (size_t)nvshmemi_threadgroup_size<SCOPE>() &&
           ((((uintptr_t)dest) | (uintptr_t)source) & 15) == 0 && (!SCATTER || (nbytes & 15) == 0);
}
NVSHMEMI_DEVICE_INLINE char *nvshmemi_amd_stage_buffer(nvshmem_team_t team, int pe, unsigned which) {
    const size_t npes = (size_t)nvshmemi_device_state_d.npes;
    return nvshmemi_device_state_d.ll_buffers +
           (size_t)NVSHMEMI_AMD_MAX_TEAMS * npes * NVSHMEMI_AMD_LL_BUFFERS * 2 * NVSHMEMI_AMD_LL_PAYLOAD_BYTES +
           (((size_t)team * npes + (size_t)pe) * NVSHMEMI_AMD_STAGE_BUFFERS + which) * NVSHMEMI_AMD_STAGE_BYTES;
}
template <typename T, int OP, int SCOPE, bool SCATTER>
NVSHMEMI_DEVICE_INLINE void nvshmemi_amd_staged_reduce(nvshmem_team_t team, const nvshmemi_amd_team_view_t &tv,
                                                       T *dest, const T *source, size_t nreduce) {
    constexpr size_t VEC = 16 / sizeof(T);
    struct alignas(16) pack_t { T e[VEC]; };
    const int me = tv.my_pe, npes = tv.size;
    const size_t tid = (size_t)nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const size_t nthr = (size_t)nvshmemi_threadgroup_size<SCOPE>();
    const size_t nbytes = nreduce * sizeof(T);
    const size_t slot = (nbytes + 15) & ~(size_t)15;
    const size_t nvec = nreduce / VEC;
    nvshmemi_threadgroup_sync<SCOPE>();
    const uint64_t before =
        *reinterpret_cast<volatile uint64_t *>(nvshmemi_amd_sync_epoch(team, nvshmemi_amd_my_pe()));
    const unsigned which = (unsigned)(before & 1);
    const T *src = reinterpret_cast<const T *>(nvshmemi_amd_local(source));
    /* push: member idx gets src (SCATTER: block idx of src) in slot me */
    for (size_t v = tid; v < nvec; v += nthr) {
        /* (plain 16-byte vectors: as an array of the element union the batch was kept in scratch memory) */
        for (int i0 = 0; i0 < npes; i0 += 8) {
            nvshmemi_v4u x[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int ii = i0 + k < npes ? i0 + k : npes - 1; /* past the end: the last member once more */
                const int idx = me + ii < npes ? me + ii : me + ii - npes;
                if (SCATTER || k == 0)
                    x[k] = *reinterpret_cast<const nvshmemi_v4u *>(src + (SCATTER ? (size_t)idx * nreduce : 0) + v * VEC);
                else
                    x[k] = x[0];
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int ii = i0 + k < npes ? i0 + k : npes - 1;
                const int idx = me + ii < npes ? me + ii : me + ii - npes;
                char *to = nvshmemi_amd_stage_buffer(team, nvshmemi_amd_team_pe(tv, idx), which) + (size_t)me * slot;
                *reinterpret_cast<nvshmemi_v4u *>(to + 16 * v) = x[k];
            }
        }
    }
    for (size_t i = nvec * VEC + tid; i < nreduce; i += nthr) /* not SCATTER: its blocks are whole vectors */
        for (int ii = 0; ii < npes; ++ii) {
            const int idx = me + ii < npes ? me + ii : me + ii - npes;
            char *to = nvshmemi_amd_stage_buffer(team, nvshmemi_amd_team_pe(tv, idx), which) + (size_t)me * slot;
            reinterpret_cast<T *>(to)[i] = src[i];
        }
    nvshmemi_quiet<SCOPE>();
    nvshmemi_amd_sync_arrive_wait<SCOPE>(team, tv, before + 1);
    /* fold my copy of everybody's contribution */
    const char *mine = nvshmemi_amd_stage_buffer(team, nvshmemi_amd_my_pe(), which);
    T *dst = reinterpret_cast<T *>(nvshmemi_amd_local(dest));
    for (size_t v = tid; v < nvec; v += nthr) {
        pack_t acc;
        for (int p0 = 0; p0 < npes; p0 += 8) {
            pack_t x[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int pe = p0 + k < npes ? p0 + k : npes - 1;
                x[k] = *reinterpret_cast<const pack_t *>(mine + (size_t)pe * slot + 16 * v);
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int pe = p0 + k;
                if (pe == 0) acc = x[0];
                else if (pe < npes) {
#pragma unroll
                    for (size_t e = 0; e < VEC; ++e)
                        acc.e[e] = SCATTER ? nvshmemi_amd_reduce_op<T, OP>(acc.e[e], x[k].e[e])
                                           : nvshmemi_amd_fold_step<T, OP>(pe, acc.e[e], x[k].e[e]);
                }
            }
        }
        *reinterpret_cast<pack_t *>(dst + v * VEC) = acc;
    }
    for (size_t i = nvec * VEC + tid; i < nreduce; i += nthr) {
        T acc = reinterpret_cast<const T *>(mine)[i];
        for (int pe = 1; pe < npes; ++pe)
            acc = nvshmemi_amd_fold_step<T, OP>(pe, acc, reinterpret_cast<const T *>(mine + (size_t)pe * slot)[i]);
        dst[i] = acc;
    }
}

template <typename T, int OP, int SCOPE>
NVSHMEMI_DEVICE_INLINE int nvshmemi_reduce_threadgroup(nvshmem_team_t team, T *dest, const T *source,
                                                       size_t nreduce) {
    constexpr size_t VEC = 16 / sizeof(T);
    struct alignas(16) pack_t { T e[VEC]; };
    const nvshmemi_amd_team_view_t tv = nvshmemi_amd_team_view(team);
    if (tv.size <= 0) return 1; /* the calling PE is not a member */
    const int me = tv.my_pe;
    const int npes = tv.size;
    const size_t tid = (size_t)nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const size_t nthr = (size_t)nvshmemi_threadgroup_size<SCOPE>();
    if (const unsigned group = nvshmemi_amd_ll_reduce_group<SCOPE>(nreduce * sizeof(T), npes)) {
        nvshmemi_amd_ll_reduce<T, OP, SCOPE>(team, tv, dest, source, nreduce, group);
        return 0;
    }
#ifdef NVSHMEMI_AMD_UNIT_PACKETS
    if (nvshmemi_amd_units_fit<SCOPE>(nreduce * sizeof(T), npes)) {
        nvshmemi_amd_unit_reduce<T, OP, SCOPE, false>(team, tv, dest, source, nreduce);
        return 0;
    }
#endif
    if (nvshmemi_amd_staged_fits<SCOPE, false>(dest, source, nreduce * sizeof(T), npes)) {
        nvshmemi_amd_staged_reduce<T, OP, SCOPE, false>(team, tv, dest, source, nreduce);
        return 0;
    }
    /* every PE's source is complete and visible before anyone reads it */
    nvshmemi_barrier_threadgroup<SCOPE>(team);
    /* member 0's copies; member i's are i * pe_stride elements further */
    const T *src0 = reinterpret_cast<const T *>(nvshmemi_amd_remote(source, tv.start));
    T *dst0 = reinterpret_cast<T *>(nvshmemi_amd_remote(dest, tv.start));
    const size_t pe_stride = (size_t)(nvshmemi_device_state_d.heap_size / sizeof(T)) * (size_t)tv.stride;
    const bool vectors = (((uintptr_t)src0 | (uintptr_t)dst0) & 15) == 0;
    /* chunk in elements, a whole number of vectors on the vector path */
    size_t chunk = (nreduce + (size_t)npes - 1) / (size_t)npes;
    if (vectors) chunk = (chunk + VEC - 1) / VEC * VEC;
    size_t lo = (size_t)me * chunk;
    if (lo > nreduce) lo = nreduce;
    size_t hi = lo + chunk;
    if (hi > nreduce) hi = nreduce;
    size_t i = lo + tid;
    if (vectors) {
        const size_t nvec = (hi - lo) / VEC;
        for (size_t v = tid; v < nvec; v += nthr) {
            const size_t at = lo + v * VEC;
            /* the members' vectors are fetched eight at a time, all loads before the first fold: one
             * after the other they would each pay the way to another PE's memory */
            pack_t acc;
            for (int p0 = 0; p0 < npes; p0 += 8) {
                pack_t x[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int pe = p0 + k < npes ? p0 + k : npes - 1; /* past the end: fetched again, not folded */
                    x[k] = *reinterpret_cast<const pack_t *>(src0 + (size_t)pe * pe_stride + at);
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int pe = p0 + k;
                    if (pe == 0) acc = x[0];
                    else if (pe < npes) {
#pragma unroll
                        for (size_t e = 0; e < VEC; ++e) acc.e[e] = nvshmemi_amd_fold_step<T, OP>(pe, acc.e[e], x[k].e[e]);
                    }
                }
            }
            for (int pe = 0; pe < npes; ++pe)
                *reinterpret_cast<pack_t *>(dst0 + (size_t)pe * pe_stride + at) = acc;
        }
        i = lo + nvec * VEC + tid; /* the last PE's range may end inside a vector */
    }
    for (; i < hi; i += nthr) {
        const T acc = nvshmemi_amd_fold_element<T, OP>(src0, pe_stride, npes, i);
        for (int pe = 0; pe < npes; ++pe) dst0[(size_t)pe * pe_stride + i] = acc;
    }
    nvshmemi_barrier_threadgroup<SCOPE>(team);
    return 0;
}

template <typename T, int SCOPE>
NVSHMEMI_DEVICE_INLINE int nvshmemi_fcollect_threadgroup(nvshmem_team_t team, T *dest,
                                                         const T *source, size_t nelems) {
    const nvshmemi_amd_team_view_t tv = nvshmemi_amd_team_view(team);
    if (tv.size <= 0) return 1;
    const int me = tv.my_pe;
    const int npes = tv.size;
    const size_t nbytes = nelems * sizeof(T);
    if (nvshmemi_amd_ll_fits<SCOPE>(nbytes, npes)) {
        /* small contributions: packets to every member's buffer, then unpack what arrived here;
         * the (member, chunk) pairs are spread over the lanes both ways */
        const unsigned tid = (unsigned)nvshmemi_thread_id_in_threadgroup<SCOPE>();
        const unsigned nthr = (unsigned)nvshmemi_threadgroup_size<SCOPE>();
        const uint32_t flag = nvshmemi_amd_ll_next_flag<SCOPE>(team);
        const unsigned npk = nvshmemi_amd_ll_packets(nbytes);
        const unsigned total = (unsigned)(npes - 1) * npk;
        const char *src = nvshmemi_amd_local(source);
        char *dst = nvshmemi_amd_local(dest);
        nvshmemi_amd_ll_send_to_all<SCOPE>(team, tv, src, nbytes, npk, (unsigned)me * npk, flag);
        /* the caller's own block: a single thread moves it eight bytes at a time (byte by byte every
         * store waited for a load), the lanes of a group a byte each */
        if (SCOPE == NVSHMEMI_THREADGROUP_THREAD)
            for (unsigned j = 0; j < npk; ++j)
                nvshmemi_amd_ll_store_payload(dst + (size_t)me * nbytes + 8 * (size_t)j,
                                              nvshmemi_amd_ll_load_payload(src + 8 * (size_t)j, nbytes - 8 * (size_t)j),
                                              nbytes - 8 * (size_t)j);
        else
            for (size_t b = tid; b < nbytes; b += nthr) dst[(size_t)me * nbytes + b] = src[b];
        const char *mine = nvshmemi_amd_ll_buffer(team, nvshmemi_amd_my_pe(), flag);
        for (unsigned w = tid; w < total; w += nthr) {
            const unsigned off = w / npk, j = w - off * npk;
            int idx = me + 1 + (int)off;
            if (idx >= npes) idx -= npes;
            const uint64_t v = nvshmemi_amd_ll_recv_packet(mine + ((size_t)idx * npk + j) * 16, flag);
            nvshmemi_amd_ll_store_payload(dst + (size_t)idx * nbytes + 8 * (size_t)j, v, nbytes - 8 * (size_t)j);
        }
        nvshmemi_amd_ll_publish_done<SCOPE>(team, flag);
        return 0;
    }
    nvshmemi_threadgroup_sync<SCOPE>();
    if (!nvshmemi_amd_fanout_copy<SCOPE>(tv, dest + (size_t)me * nelems, nvshmemi_amd_local(source), 0, nbytes))
        for (int ii = 0; ii < npes; ++ii) {
            const int peer = nvshmemi_amd_team_pe(tv, (me + ii) % npes);
            nvshmemi_memcpy_threadgroup<SCOPE>(nvshmemi_amd_remote(dest + (size_t)me * nelems, peer),
                                               nvshmemi_amd_local(source), nelems * sizeof(T));
        }
    nvshmemi_barrier_threadgroup<SCOPE>(team);
    return 0;
}

template <typename T, int SCOPE>
NVSHMEMI_DEVICE_INLINE int nvshmemi_alltoall_threadgroup(nvshmem_team_t team, T *dest,
                                                         const T *source, size_t nelems) {
    const nvshmemi_amd_team_view_t tv = nvshmemi_amd_team_view(team);
    if (tv.size <= 0) return 1;
    const int me = tv.my_pe;
    const int npes = tv.size;
    const size_t nbytes = nelems * sizeof(T);
    if (nvshmemi_amd_ll_fits<SCOPE>(nbytes, npes)) {
        /* small blocks: like the fcollect packets, but member idx is sent block idx */
        const unsigned tid = (unsigned)nvshmemi_thread_id_in_threadgroup<SCOPE>();
        const unsigned nthr = (unsigned)nvshmemi_threadgroup_size<SCOPE>();
        const uint32_t flag = nvshmemi_amd_ll_next_flag<SCOPE>(team);
        const unsigned npk = nvshmemi_amd_ll_packets(nbytes);
        const unsigned total = (unsigned)(npes - 1) * npk;
        const char *src = nvshmemi_amd_local(source);
        char *dst = nvshmemi_amd_local(dest);
        nvshmemi_amd_ll_send_to_all<SCOPE>(team, tv, src, nbytes, npk, (unsigned)me * npk, flag, nbytes);
        if (SCOPE == NVSHMEMI_THREADGROUP_THREAD)
            for (unsigned j = 0; j < npk; ++j)
                nvshmemi_amd_ll_store_payload(
                    dst + (size_t)me * nbytes + 8 * (size_t)j,
                    nvshmemi_amd_ll_load_payload(src + (size_t)me * nbytes + 8 * (size_t)j, nbytes - 8 * (size_t)j),
                    nbytes - 8 * (size_t)j);
        else
            for (size_t b = tid; b < nbytes; b += nthr) dst[(size_t)me * nbytes + b] = src[(size_t)me * nbytes + b];
        const char *mine = nvshmemi_amd_ll_buffer(team, nvshmemi_amd_my_pe(), flag);
        for (unsigned w = tid; w < total; w += nthr) {
            const unsigned off = w / npk, j = w - off * npk;
            int idx = me + 1 + (int)off;
            if (idx >= npes) idx -= npes;
            const uint64_t v = nvshmemi_amd_ll_recv_packet(mine + ((size_t)idx * npk + j) * 16, flag);
            nvshmemi_amd_ll_store_payload(dst + (size_t)idx * nbytes + 8 * (size_t)j, v, nbytes - 8 * (size_t)j);
        }
        nvshmemi_amd_ll_publish_done<SCOPE>(team, flag);
        return 0;
    }
    nvshmemi_threadgroup_sync<SCOPE>();
    if (!nvshmemi_amd_fanout_copy<SCOPE>(tv, dest + (size_t)me * nelems, nvshmemi_amd_local(source), nbytes, nbytes))
        for (int ii = 0; ii < npes; ++ii) {
            const int idx = (me + ii) % npes;
            nvshmemi_memcpy_threadgroup<SCOPE>(
                nvshmemi_amd_remote(dest + (size_t)me * nelems, nvshmemi_amd_team_pe(tv, idx)),
                nvshmemi_amd_local(source + (size_t)idx * nelems), nelems * sizeof(T));
        }
    nvshmemi_barrier_threadgroup<SCOPE>(team);
    return 0;
}

/* Broadcast (reference coll/broadcast.cuh:298-337, the put-to-all algorithm): the root's thread
 * group copies its source into every member's dest, its own included unless dest == source; the
 * closing barrier completes the copies and tells the receivers.  PE_root is an index of the team. */
template <typename T, int SCOPE>
NVSHMEMI_DEVICE_INLINE int nvshmemi_broadcast_threadgroup(nvshmem_team_t team, T *dest,
                                                          const T *source, size_t nelems,
                                                          int PE_root) {
    const nvshmemi_amd_team_view_t tv = nvshmemi_amd_team_view(team);
    if (tv.size <= 0) return 1;
    const int me = tv.my_pe;
    const int npes = tv.size;
    const size_t nbytes = nelems * sizeof(T);
    /* a single thread also sends one after the other, so all its packets count */
    /* ... and where the fan-out copy applies, the packets are taken only while the root's (member, chunk)
     * pairs fit one round of stores over its lanes: every further round costs 0.4-0.5 us (8 PEs, 256
     * threads: 1.65 us with one round, 2.2-2.4 with two, 2.6 with three), the fan-out copy and its
     * barrier 2.1-2.3 us flat up to 4 KiB */
    if (nbytes > 0 && nbytes <= NVSHMEMI_AMD_LL_BCAST_MAX_BYTES && nvshmemi_amd_ll_available() &&
        ((nbytes + 7) >> 3) * (size_t)(SCOPE == NVSHMEMI_THREADGROUP_THREAD ? npes - 1 : 1) <=
            nvshmemi_amd_ll_lanes<SCOPE>() &&
        (((nbytes + 7) >> 3) * (size_t)(npes - 1) <= (size_t)nvshmemi_amd_ll_lanes<SCOPE>() ||
         !nvshmemi_amd_fanout_fits<SCOPE>(dest, source, 0, nbytes))) {
        const unsigned tid = (unsigned)nvshmemi_thread_id_in_threadgroup<SCOPE>();
        const unsigned nthr = (unsigned)nvshmemi_threadgroup_size<SCOPE>();
        const uint32_t flag = nvshmemi_amd_ll_next_flag<SCOPE>(team);
        const unsigned npk = nvshmemi_amd_ll_packets(nbytes);
        if (me == PE_root) {
            const char *src = nvshmemi_amd_local(source);
            char *dst = nvshmemi_amd_local(dest);
            /* nothing else orders a root against its receivers: all of them must have finished
             * reading call flag - 2 before anybody may be sent call flag */
            if (flag > 2 && nthr >= (unsigned)npes) {
                if (tid < (unsigned)npes && (int)tid != me)
                    nvshmemi_wait_until<uint64_t>(
                        nvshmemi_amd_ll_word(team, nvshmemi_amd_team_pe(tv, (int)tid), NVSHMEMI_AMD_LL_DONE_WORD),
                        NVSHMEM_CMP_GE, (uint64_t)(flag - 2));
            } else if (flag > 2) {
                /* a lane that answers for several members reads eight of their words per round trip (the
                 * root's own word is past flag - 2 as well, so nobody is left out) */
                const uint64_t limit = nvshmemi_device_state_d.spin_limit;
                uint64_t polls = 0;
                for (;;) {
                    uint64_t lowest = ~(uint64_t)0;
                    for (unsigned i0 = tid; i0 < (unsigned)npes; i0 += 8 * nthr) {
                        uint64_t x[8];
#pragma unroll
                        for (unsigned k = 0; k < 8; ++k) {
                            const unsigned i = i0 + k * nthr < (unsigned)npes ? i0 + k * nthr : i0;
                            x[k] = nvshmemi_amd_poll(reinterpret_cast<const uint64_t *>(
                                nvshmemi_amd_ll_word(team, nvshmemi_amd_team_pe(tv, (int)i), NVSHMEMI_AMD_LL_DONE_WORD)));
                        }
#pragma unroll
                        for (unsigned k = 0; k < 8; ++k) lowest = x[k] < lowest ? x[k] : lowest;
                    }
                    if (lowest >= (uint64_t)(flag - 2)) break;
                    if (limit && ++polls > limit) {
                        nvshmemi_amd_record_timeout(
                            nvshmemi_amd_ll_word(team, nvshmemi_amd_team_pe(tv, (int)tid), NVSHMEMI_AMD_LL_DONE_WORD), lowest,
                            (uint64_t)(flag - 2));
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
            }
            nvshmemi_threadgroup_sync<SCOPE>();
            nvshmemi_amd_ll_send_to_all<SCOPE>(team, tv, src, nbytes, npk, 0, flag);
            if (dst != src)
                for (size_t b = tid; b < nbytes; b += nthr) dst[b] = src[b];
        } else {
            char *dst = nvshmemi_amd_local(dest);
            const char *mine = nvshmemi_amd_ll_buffer(team, nvshmemi_amd_my_pe(), flag);
            for (unsigned j = tid; j < npk; j += nthr)
                nvshmemi_amd_ll_store_payload(dst + 8 * (size_t)j, nvshmemi_amd_ll_recv_packet(mine + (size_t)j * 16, flag),
                                              nbytes - 8 * (size_t)j);
        }
        nvshmemi_amd_ll_publish_done<SCOPE>(team, flag);
        return 0;
    }
    if (nbytes >= NVSHMEMI_AMD_BCAST_PULL_BYTES ||
        nbytes >= (size_t)NVSHMEMI_AMD_BCAST_PULL_BYTES_PER_LANE * (size_t)nvshmemi_threadgroup_size<SCOPE>()) {
        /* long messages: a root that pushes does all the work alone (1 MiB to 8 PEs from one block:
         * 98 us).  Instead everybody meets - the root's source is complete and written back by then -
         * and every PE fetches the message itself, all blocks at once (17 us), and meets again, after
         * which the root may reuse its source.  Two barriers instead of one pay off from 32 KiB on for a
         * block and from 128 bytes per lane for smaller groups (a wavefront: 8 KiB, 4.5 against 5.3 us). */
        nvshmemi_barrier_threadgroup<SCOPE>(team);
        const char *from = nvshmemi_amd_remote(source, nvshmemi_amd_team_pe(tv, PE_root));
        char *to = nvshmemi_amd_local(dest);
        if (to != from) nvshmemi_memcpy_threadgroup<SCOPE>(to, from, nbytes);
        nvshmemi_barrier_threadgroup<SCOPE>(team);
        return 0;
    }
    if (me == PE_root) {
        const void *from = nvshmemi_amd_local(source);
        /* (the fan-out rewrites the root's own bytes with themselves when dest is source there) */
        if (!nvshmemi_amd_fanout_copy<SCOPE>(tv, dest, (const char *)from, 0, nelems * sizeof(T)))
            for (int ii = 0; ii < npes; ++ii) {
                void *to = nvshmemi_amd_remote(dest, nvshmemi_amd_team_pe(tv, (me + ii) % npes));
                if (to != from) nvshmemi_memcpy_threadgroup<SCOPE>(to, from, nelems * sizeof(T));
            }
    }
    nvshmemi_barrier_threadgroup<SCOPE>(team);
    return 0;
}

/* Reducescatter (reference coll/reducescatter.cuh:36-90): member `me` folds block `me` (nreduce
 * elements) of every member's source into its own dest, in the order acc = op(x0, x1);
 * acc = op(acc, x_p).  dest must not overlap source: other PEs read the blocks of this PE's source
 * while it writes its dest. */
template <typename T, int OP, int SCOPE>
NVSHMEMI_DEVICE_INLINE int nvshmemi_reducescatter_threadgroup(nvshmem_team_t team, T *dest,
                                                              const T *source, size_t nreduce) {
    constexpr size_t VEC = 16 / sizeof(T);
    struct alignas(16) pack_t { T e[VEC]; };
    const nvshmemi_amd_team_view_t tv = nvshmemi_amd_team_view(team);
    if (tv.size <= 0) return 1;
    const int me = tv.my_pe;
    const int npes = tv.size;
    const size_t tid = (size_t)nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const size_t nthr = (size_t)nvshmemi_threadgroup_size<SCOPE>();
    if (const unsigned group = nvshmemi_amd_ll_reduce_group<SCOPE>(nreduce * sizeof(T), npes)) {
        nvshmemi_amd_ll_reduce<T, OP, SCOPE, true>(team, tv, dest, source, nreduce, group);
        return 0;
    }
#ifdef NVSHMEMI_AMD_UNIT_PACKETS
    if (nvshmemi_amd_units_fit<SCOPE>(nreduce * sizeof(T), npes)) {
        nvshmemi_amd_unit_reduce<T, OP, SCOPE, true>(team, tv, dest, source, nreduce);
        return 0;
    }
#endif
    if (nvshmemi_amd_staged_fits<SCOPE, true>(dest, source, nreduce * sizeof(T), npes)) {
        nvshmemi_amd_staged_reduce<T, OP, SCOPE, true>(team, tv, dest, source, nreduce);
        return 0;
    }
    /* every PE's source is complete and visible before anyone reads it */
    nvshmemi_barrier_threadgroup<SCOPE>(team);
    const T *src0 = reinterpret_cast<const T *>(nvshmemi_amd_remote(source, tv.start)) + (size_t)me * nreduce;
    T *dst = reinterpret_cast<T *>(nvshmemi_amd_remote(dest, nvshmemi_amd_my_pe()));
    const size_t pe_stride = (size_t)(nvshmemi_device_state_d.heap_size / sizeof(T)) * (size_t)tv.stride;
    size_t i = tid;
    if ((((uintptr_t)src0 | (uintptr_t)dst) & 15) == 0) {
        const size_t nvec = nreduce / VEC;
        for (size_t v = tid; v < nvec; v += nthr) {
            /* eight members' vectors are fetched before the first fold, as in the allreduce */
            pack_t acc;
            for (int p0 = 0; p0 < npes; p0 += 8) {
                pack_t x[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int pe = p0 + k < npes ? p0 + k : npes - 1;
                    x[k] = *reinterpret_cast<const pack_t *>(src0 + (size_t)pe * pe_stride + v * VEC);
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int pe = p0 + k;
                    if (pe == 0) acc = x[0];
                    else if (pe < npes) {
#pragma unroll
                        for (size_t e = 0; e < VEC; ++e) acc.e[e] = nvshmemi_amd_reduce_op<T, OP>(acc.e[e], x[k].e[e]);
                    }
                }
            }
            *reinterpret_cast<pack_t *>(dst + v * VEC) = acc;
        }
        i = nvec * VEC + tid;
    }
    for (; i < nreduce; i += nthr) {
        T acc = src0[i];
        for (int pe = 1; pe < npes; ++pe)
            acc = nvshmemi_amd_reduce_op<T, OP>(acc, src0[(size_t)pe * pe_stride + i]);
        dst[i] = acc;
    }
    nvshmemi_barrier_threadgroup<SCOPE>(team);
    return 0;
}

/* maxloc on (value, location) pairs (reference reduce.cuh:107-111 and :1718-1751): every member's
 * dest[i] = fold over the members 0..n-1 of source[i], acc = (acc.x > x.x) ? acc : x - the order of the
 * reference's rooted flat reduce, whose result all members then share: on equal values the later
 * member wins, and a NaN met as x replaces acc.  The reference takes one element per call; any
 * nreduce is served here.  Every member folds all elements itself and writes only its own dest. */
NVSHMEMI_DEVICE_INLINE int nvshmemi_double2_maxloc_reduce_block(nvshmem_team_t team, double2 *dest,
                                                               const double2 *source, size_t nreduce) {
    constexpr int SCOPE = NVSHMEMI_THREADGROUP_BLOCK;
    const nvshmemi_amd_team_view_t tv = nvshmemi_amd_team_view(team);
    if (tv.size <= 0) return 1; /* the calling PE is not a member */
    const size_t tid = (size_t)nvshmemi_thread_id_in_threadgroup<SCOPE>();
    const size_t nthr = (size_t)nvshmemi_threadgroup_size<SCOPE>();
    double2 *dst = reinterpret_cast<double2 *>(nvshmemi_amd_remote(dest, nvshmemi_amd_my_pe()));
    /* One pair per PE, the reference's case: every member sends its pair to all others as two
     * packets and folds what it receives.  Lane (j, p) of the first wavefront holds word j (0: value,
     * 1: location) of member p, so the fold reads its operands across lanes instead of polling
     * packet after packet. */
    unsigned group = 1;
    while ((int)group < tv.size) group <<= 1;
    if (nreduce == 1 && 2 * group <= 64 && nthr >= 64 && nvshmemi_amd_ll_fits<SCOPE>(sizeof(double2), tv.size)) {
        const int me = tv.my_pe;
        const uint32_t flag = nvshmemi_amd_ll_next_flag<SCOPE>(team);
        const char *src = nvshmemi_amd_local(source);
        nvshmemi_amd_ll_send_to_all<SCOPE>(team, tv, src, sizeof(double2), 2, (unsigned)me * 2, flag);
        nvshmemi_threadgroup_sync<SCOPE>(); /* dest may be source: sent before the result is stored */
        if (tid < 64) {
            const char *mine = nvshmemi_amd_ll_buffer(team, nvshmemi_amd_my_pe(), flag);
            const unsigned gshift = 31u - (unsigned)__builtin_clz(group);
            const unsigned j = (unsigned)tid >> gshift, p = (unsigned)tid & (group - 1);
            uint64_t v = 0;
            if (j < 2 && (int)p < tv.size)
                v = (int)p == me ? nvshmemi_amd_ll_load_payload(src + 8 * (size_t)j, 8)
                                 : nvshmemi_amd_ll_recv_packet(mine + ((size_t)p * 2 + j) * 16, flag);
            uint64_t best_v = 0, best_l = 0;
            for (int q = 0; q < tv.size; ++q) {
                const uint64_t xv = (uint64_t)__shfl((unsigned long long)v, q, 64);
                const uint64_t xl = (uint64_t)__shfl((unsigned long long)v, (int)group + q, 64);
                double a, b;
                __builtin_memcpy(&a, &best_v, 8);
                __builtin_memcpy(&b, &xv, 8);
                if (q == 0 || !(a > b)) {
                    best_v = xv;
                    best_l = xl;
                }
            }
            if (tid == 0) {
                nvshmemi_amd_ll_store_payload(reinterpret_cast<char *>(dst), best_v, 8);
                nvshmemi_amd_ll_store_payload(reinterpret_cast<char *>(dst) + 8, best_l, 8);
            }
        }
        nvshmemi_amd_ll_publish_done<SCOPE>(team, flag);
        return 0;
    }
    /* every PE's source is complete and visible before anyone reads it */
    nvshmemi_barrier_threadgroup<SCOPE>(team);
    const double2 *src0 = reinterpret_cast<const double2 *>(nvshmemi_amd_remote(source, tv.start));
    const size_t pe_stride = (size_t)(nvshmemi_device_state_d.heap_size / sizeof(double2)) * (size_t)tv.stride;
    for (size_t i = tid; i < nreduce; i += nthr) {
        double2 acc = src0[i];
        for (int pe = 1; pe < tv.size; ++pe) {
            const double2 x = src0[(size_t)pe * pe_stride + i];
            acc = (acc.x > x.x) ? acc : x;
        }
        dst[i] = acc;
    }
    /* nobody may overwrite its source before every member has read it */
    nvshmemi_barrier_threadgroup<SCOPE>(team);
    return 0;
}

#endif
