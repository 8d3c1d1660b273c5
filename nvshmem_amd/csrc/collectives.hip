// Host-launched collectives for logical PEs on one MI355X: one grid-wide kernel per call serves
// every PE of the team - and, when the handle names a family of disjoint teams (the rows of a 2-D
// split), every team of the family: grid.z indexes the team, whose <start, stride, size> the kernel
// reads from the device copy of the team table.
//
// Reference counterparts: the on-stream launchers src/host/stream/coll/{rdxn/reduce_common.cuh:29-68,
// fcollect/fcollect.cu:20-65, alltoall/alltoall.cu:18-40} start one block per PE that runs the
// device templates coll/reduce.cuh:1592-1674, coll/fcollect.cuh:331-344, coll/alltoall.cuh:122-143
// and meets the other PEs in a flag barrier.  Here all PEs share one HBM, so a collective is a
// single streaming pass: every source byte is read once, every destination byte written once, and
// the kernel boundary is the barrier.
//
//   reduce    dest@q[k] = fold_{p = 0..n-1, in that order} src@p[k]      for every PE q
//   fcollect  dest@q[p*nelems + k] = src@p[k]                            for every PE q
//   alltoall  dest@q[p*nelems + k] = src@p[q*nelems + k]
//   broadcast dest@q[k] = src@root[k]                                    for every PE q
//   reducescatter  dest@q[k] = fold_{p = 0..n-1} src@p[q*nreduce + k]
//
// Reference counterparts of the last two: src/host/coll/broadcast/broadcast.cpp with
// coll/broadcast.cuh:276-337, src/host/coll/reducescatter/reducescatter_on_stream.cpp with
// coll/reducescatter.cuh:36-90.
#include <cstdio>

#include "nvshmem.h"
#include "runtime.hpp"

namespace nvshmem_amd {
namespace {

// Tunables (compile time).  Defaults are the values measured best on MI355X.
#ifndef NVSHMEM_AMD_COLL_THREADS
#define NVSHMEM_AMD_COLL_THREADS 256
#endif
#ifndef NVSHMEM_AMD_COPY_THREADS /* threads per block of the segment copy: one wavefront */
#define NVSHMEM_AMD_COPY_THREADS 64
#endif
#ifndef NVSHMEM_AMD_ALLTOALL_UNROLL /* vectors per lane in an alltoall tile */
#define NVSHMEM_AMD_ALLTOALL_UNROLL 1
#endif
#ifndef NVSHMEM_AMD_FCOLLECT_UNROLL /* vectors per lane in an fcollect tile */
#define NVSHMEM_AMD_FCOLLECT_UNROLL 1
#endif
#ifndef NVSHMEM_AMD_REDUCE_VPT /* vectors a thread of the fused reduce loads per tile */
#define NVSHMEM_AMD_REDUCE_VPT 1
#endif
#ifndef NVSHMEM_AMD_REDUCE_VPT_NARROW /* the same for 1- and 2-byte elements on the compile-time team sizes 8 and 16 */
#define NVSHMEM_AMD_REDUCE_VPT_NARROW 1
#endif
/* Members per wavefront of the fused reduce on the compile-time team sizes 8 and 16, for 1- and 2-byte
 * elements (NARROW) and for wider ones (WIDE).  Narrow elements fold twice to four times as many elements
 * per byte, and a block has nothing in flight while it folds: with two members per wavefront the blocks
 * are half as large and twice as many share a compute unit, so more of them are in their load or store
 * phase at any time (bf16 sum and max, 8 x 128 MiB: 6.05-6.15 TB/s with one member per wavefront and two
 * vectors per thread, 6.21-6.25 with two members and one vector; four members 5.74-5.96).  4- and 8-byte
 * elements lose 5 % with two members per wavefront and 11 % with four. */
#ifndef NVSHMEM_AMD_REDUCE_NARROW_MPW
#define NVSHMEM_AMD_REDUCE_NARROW_MPW 2
#endif
#ifndef NVSHMEM_AMD_REDUCE_WIDE_MPW
#define NVSHMEM_AMD_REDUCE_WIDE_MPW 1
#endif
#ifndef NVSHMEM_AMD_COLL_NT /* bit 0: non-temporal loads allowed, bit 1: non-temporal stores */
#define NVSHMEM_AMD_COLL_NT 3
#endif
/* Sources of up to Runtime::cacheable_source_bytes (all PEs together, 256 MiB unless the environment
 * says otherwise) are loaded with the default, cacheable policy: they fit the 256 MiB Infinity
 * Cache, so a source that is sent again (or was just produced) is served from it (measured +30 % on
 * the 1M-element reduce, +20..45 % on 256 MiB collectives).  Larger sources are streamed with
 * non-temporal loads (+5 % at 2 GiB).  Stores always stream. */

constexpr int kThreads = NVSHMEM_AMD_COLL_THREADS;
constexpr int kCopyThreads = NVSHMEM_AMD_COPY_THREADS;

template <bool NTL>
__device__ __forceinline__ nvshmemi_v4u stream_load(const char *p) {
    if (NTL && (NVSHMEM_AMD_COLL_NT & 1))
        return __builtin_nontemporal_load(reinterpret_cast<const nvshmemi_v4u *>(p));
    return *reinterpret_cast<const nvshmemi_v4u *>(p);
}
// How a kernel's result stores treat the caches.  All three stream (nothing here reads its output back);
// they differ in where the line waits for memory.  Write-through stores (sc1) leave the L2 at once
// instead of queuing behind its eviction of streaming lines: a write-only stream reaches 7.2 TB/s with
// them against 6.3 TB/s with nt alone.  Which form wins depends on the kernel's mix (measured on MI355X,
// random data): sc1 nt +4.5 % for the 8-member allreduce, +5..10 % for fcollect and cache-resident
// broadcast, +1..3 % for alltoall and the gather allreduce; plain sc1 +5 % for the reducescatter, whose
// one store per eight loads gains nothing from nt; and the kernels whose blocks share a piece through
// the cache (destinations split over neighbouring blocks) lose 9..15 % with either, so they keep nt.
enum { kStoreStream = 0 /* nt */, kStoreThrough = 1 /* sc1 */, kStoreThroughStream = 2 /* sc1 nt */ };
#ifndef NVSHMEM_AMD_STORE_ALLTOALL
#define NVSHMEM_AMD_STORE_ALLTOALL kStoreThroughStream
#endif
#ifndef NVSHMEM_AMD_STORE_REPLICATE /* fcollect and broadcast, one wavefront storing to every member */
#define NVSHMEM_AMD_STORE_REPLICATE kStoreThroughStream
#endif
#ifndef NVSHMEM_AMD_STORE_REDUCE
#define NVSHMEM_AMD_STORE_REDUCE kStoreThroughStream
#endif
#ifndef NVSHMEM_AMD_STORE_REDUCESCATTER
#define NVSHMEM_AMD_STORE_REDUCESCATTER kStoreThrough
#endif
// The asm forms end in s_nop 1: the compiler does not know the statement is a store of more than 8 bytes
// and would not keep the wait state this GPU needs before the data registers are written again.
template <int STORE>
__device__ __forceinline__ void stream_store(char *p, nvshmemi_v4u v) {
    if (STORE == kStoreThrough)
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
    else if (STORE == kStoreThroughStream)
        asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
    else if (NVSHMEM_AMD_COLL_NT & 2)
        __builtin_nontemporal_store(v, reinterpret_cast<nvshmemi_v4u *>(p));
    else
        *reinterpret_cast<nvshmemi_v4u *>(p) = v;
}

// ---------------------------------------------------------------------------------------------
// Segment copy: fcollect and alltoall are sets of contiguous (source, destination) segments.
// grid.y indexes the segment, grid.x the tile inside it.  A block is ONE wavefront that moves ONE
// aligned 1 KiB piece (64 lanes x 16 bytes): on MI355X this shape measured fastest by a clear
// margin (6.7-6.8 TB/s for alltoall, against 6.0 TB/s with 256-thread blocks and 8 KiB tiles and
// 4.0 TB/s with 32 KiB tiles), because the blocks in flight then cover a narrow, moving window of
// addresses.  The destination is written with aligned vectors only: block 0 of a segment copies
// the byte head in front of the first aligned destination vector and the byte tail behind the
// last one.
// ---------------------------------------------------------------------------------------------

enum { kModeFcollect = 0, kModeAlltoall = 1, kModeBroadcast = 2 };

// Copies the vectors v0 + t + u*kCopyThreads (u < unroll) that fall inside [0, nvec); indices in front of
// the segment wrap to huge unsigned values and are skipped the same way as those behind it.
template <bool SRC_ALIGNED, bool REPLICATE, int kCopyUnroll, bool NTL, int STORE>
__device__ __forceinline__ void copy_tile(char *__restrict__ dst, const char *__restrict__ src,
                                          uint64_t v0, uint64_t nvec, uint64_t rep_stride, int r0,
                                          int r1) {
    nvshmemi_v4u v[kCopyUnroll];
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) {
        const uint64_t i = v0 + threadIdx.x + (uint64_t)u * kCopyThreads;
        if (i < nvec) v[u] = SRC_ALIGNED ? stream_load<NTL>(src + 16 * i) : nvshmemi_amd_load16<false>(src + 16 * i);
    }
    if (REPLICATE) {
        for (int r = r0; r < r1; ++r) {
            char *d = dst + (uint64_t)r * rep_stride;
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u) {
                const uint64_t i = v0 + threadIdx.x + (uint64_t)u * kCopyThreads;
                if (i < nvec) stream_store<STORE>(d + 16 * i, v[u]);
            }
        }
    } else {
#pragma unroll
        for (int u = 0; u < kCopyUnroll; ++u) {
            const uint64_t i = v0 + threadIdx.x + (uint64_t)u * kCopyThreads;
            if (i < nvec) stream_store<STORE>(dst + 16 * i, v[u]);
        }
    }
}

template <int MODE, int kCopyUnroll, bool NTL, int STORE>
__global__ __launch_bounds__(kCopyThreads) void segment_copy_kernel(char *base, uint64_t slice_bytes,
                                                                const nvshmemi_amd_team_view_t *groups,
                                                                int max_size, uint64_t dst_off,
                                                                uint64_t src_off, uint64_t seg_bytes,
                                                                int root, uint32_t part_shift, uint32_t chunk_shift) {
    // this block's team: members are the PEs start + i*stride, i < size
    const nvshmemi_amd_team_view_t g = groups[blockIdx.z];
    const unsigned npes = (unsigned)g.size;
    base += (uint64_t)g.start * slice_bytes;
    const uint64_t rep_stride = (uint64_t)g.stride * slice_bytes;  // from one member to the next
    const unsigned seg = blockIdx.y;
    const char *src;
    char *dst;
    int nrep;
    if (MODE == kModeFcollect) {
        // segment p: member p's source -> slot p of every member's destination
        if (seg >= npes) return;
        src = base + seg * rep_stride + src_off;
        dst = base + dst_off + (uint64_t)seg * seg_bytes;
        nrep = (int)npes;
    } else if (MODE == kModeBroadcast) {
        // one segment: the root's source -> every member's destination
        src = base + (uint64_t)root * rep_stride + src_off;
        dst = base + dst_off;
        nrep = (int)npes;
    } else {
        // segment (p, q): block q of member p's source -> slot p of member q's destination
        const unsigned p = seg / (unsigned)max_size, q = seg % (unsigned)max_size;
        if (p >= npes || q >= npes) return;
        src = base + p * rep_stride + src_off + (uint64_t)q * seg_bytes;
        dst = base + q * rep_stride + dst_off + (uint64_t)p * seg_bytes;
        nrep = 1;
    }

    uint64_t head = (uint64_t)(-(uintptr_t)dst & 15);
    if (head > seg_bytes) head = seg_bytes;
    const uint64_t nvec_total = (seg_bytes - head) / 16;
    const uint64_t tail_start = head + nvec_total * 16;

    if (blockIdx.x == 0) {
        // at most 15 + 15 bytes per replica
        const uint64_t edge = head + (seg_bytes - tail_start);
        for (uint64_t e = threadIdx.x; e < edge * (uint64_t)nrep; e += kCopyThreads) {
            const uint64_t r = e / edge, k = e % edge;
            const uint64_t pos = k < head ? k : tail_start + (k - head);
            dst[r * rep_stride + pos] = src[pos];
        }
    }
    // tiles are cut on absolute 1 KiB boundaries of the destination: `lead` vector slots of tile 0
    // lie in front of the segment
    const uint64_t lead = ((uint64_t)(uintptr_t)(dst + head) >> 4) & 63;
    constexpr uint64_t kTileVectors = (uint64_t)kCopyThreads * kCopyUnroll;
    // fcollect / broadcast with part_shift > 0: 2^part_shift blocks share a tile and split its destinations.  The
    // sharers of a tile are 2^chunk_shift blocks apart: the grid walks a chunk of 2^chunk_shift tiles once per
    // group of destinations, so the blocks in flight write to few destinations at a time, each a run of
    // consecutive pieces, and re-read the chunk from the L2 of the XCD that fetched it (sharers are a multiple of
    // 8 blocks apart).  The host passes both shifts as zero or both as non-zero.
    uint64_t tile_index = blockIdx.x;
    unsigned part_index = 0;
    if (chunk_shift) {
        part_index = (blockIdx.x >> chunk_shift) & ((1u << part_shift) - 1);
        tile_index = (blockIdx.x & ((1u << chunk_shift) - 1)) +
                     (((uint64_t)blockIdx.x >> (chunk_shift + part_shift)) << chunk_shift);
    }
    const uint64_t v0 = tile_index * kTileVectors - lead;
    if ((int64_t)v0 >= (int64_t)nvec_total) return;
    const char *s = src + head;
    char *d = dst + head;
    const bool aligned = (((uintptr_t)s) & 15) == 0;
    if (MODE != kModeAlltoall) {
        const int per = (nrep + (1 << part_shift) - 1) >> part_shift;
        const int r0 = (int)part_index * per;
        const int r1 = r0 + per < nrep ? r0 + per : nrep;
        if (r0 >= nrep) return;  // a team smaller than the grid's largest: nothing left for this sharer
        if (aligned) copy_tile<true, true, kCopyUnroll, NTL, STORE>(d, s, v0, nvec_total, rep_stride, r0, r1);
        else copy_tile<false, true, kCopyUnroll, NTL, STORE>(d, s, v0, nvec_total, rep_stride, r0, r1);
    } else {
        if (aligned) copy_tile<true, false, kCopyUnroll, NTL, STORE>(d, s, v0, nvec_total, rep_stride, 0, 1);
        else copy_tile<false, false, kCopyUnroll, NTL, STORE>(d, s, v0, nvec_total, rep_stride, 0, 1);
    }
}

// ---------------------------------------------------------------------------------------------
// Fused reduce, LDS staged.  A block owns a tile of 64 16-byte vectors of the element range and has one
// wavefront per MPW members of the team, so a wavefront streams one aligned 1 KiB piece of a member's
// source per load.  Thread (w, i) loads vector i of the tile from members w*MPW ... w*MPW + MPW-1 into
// LDS - one load per lane and member, like a plain copy, which HBM serves measurably faster than one
// lane gathering the same vector from every PE.  After a barrier the tile's elements are folded out of
// LDS in PE order 0..n-1, one element per thread, and thread (w, i) stores result vector i into the
// destinations of its members.
// An element is read (by the loads of this block) before this block writes it and no other block
// touches it, so dest == src (in place) needs no further staging.
// ---------------------------------------------------------------------------------------------
// NPES > 0 fixes the team size at compile time (fold fully unrolled); NPES == 0 takes it from the team
// table, the block being sized for the largest team of the handle.
// fold_next: one step of the fold, in the allreduce's operand order or (SCATTER) the reducescatter's.
template <typename T, int OP, bool SCATTER>
__device__ __forceinline__ T fold_next(int p, T acc, T x) {
    return SCATTER ? nvshmemi_amd_reduce_op<T, OP>(acc, x) : nvshmemi_amd_fold_step<T, OP>(p, acc, x);
}

template <typename T, int OP, int NPES, bool NTL, int VPT = NVSHMEM_AMD_REDUCE_VPT, int MPW = 1>
__global__ __launch_bounds__(NPES ? NPES / MPW * 64 : 1024) void reduce_vector_kernel(char *base, uint64_t slice_bytes,
                                                             const nvshmemi_amd_team_view_t *groups,
                                                             uint64_t dst_off,
                                                             uint64_t src_off, uint64_t nelems) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    constexpr int VEC = 16 / sizeof(T);
    // this block's team; with NPES > 0 the host has checked that every team has NPES members
    const nvshmemi_amd_team_view_t g = groups[blockIdx.z];
    const int npes = NPES ? NPES : g.size;
    base += (uint64_t)g.start * slice_bytes;
    constexpr uint32_t lane_shift = 6;  // a wavefront's 64 lanes move one aligned 1 KiB piece of a member
    constexpr unsigned lanes = 1u << lane_shift;
    // a wavefront serves MPW consecutive members (more than one only with a compile-time team size)
    // (the wavefront's index as a scalar: the members' base addresses then stay in scalar registers)
    const unsigned pe0 = (unsigned)__builtin_amdgcn_readfirstlane(threadIdx.x >> lane_shift) * MPW,
                   i = threadIdx.x & (lanes - 1);
    const uint64_t nvec = nelems / VEC;
    // tiles are cut on absolute (16 * lanes)-byte boundaries of the destination, so a wavefront's
    // access is one aligned 1 KiB piece whatever the buffer's own alignment: `lead` vector slots of
    // the first tile lie in front of the buffer
    const uint64_t pe_stride = (uint64_t)g.stride * slice_bytes;  // from one member to the next
    // the block is sized for the largest team of the handle: lanes of members a team does not have idle
    auto member = [&](int m) { return NPES ? true : (int)pe0 + m < npes; };
    const uint64_t lead = ((uint64_t)(uintptr_t)(base + dst_off) >> 4) & (lanes - 1);
    // a tile is VPT pieces of `lanes` vectors per PE: thread (pe, i) loads vector i of each piece
    constexpr unsigned tile_vecs = (unsigned)VPT << lane_shift;
    const uint64_t ntiles = (nvec + lead + tile_vecs - 1) / tile_vecs;
    nvshmemi_v4u *stage = reinterpret_cast<nvshmemi_v4u *>(lds);           // [npes][tile_vecs]
    nvshmemi_v4u *result = stage + (size_t)npes * tile_vecs;               // [tile_vecs]
    // the unit of the fold: a 4-byte word (EPW elements) for 1- and 2-byte elements, else one element
    constexpr int EPW = sizeof(T) < 4 ? 4 / (int)sizeof(T) : 1;
    struct alignas(sizeof(T) * EPW) word_t {
        T e[EPW];
    };
    const word_t *stage_w = reinterpret_cast<const word_t *>(stage);
    word_t *result_w = reinterpret_cast<word_t *>(result);
    constexpr unsigned tile_words = tile_vecs * VEC / EPW;

    for (uint64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        // indices in front of the buffer wrap to huge values and are skipped like those behind it
        const uint64_t v0 = tile * tile_vecs + i - lead;
#pragma unroll
        for (int u = 0; u < VPT; ++u) {
            const uint64_t v = v0 + ((uint64_t)u << lane_shift);
            if (v < nvec) {
#pragma unroll
                for (int m = 0; m < MPW; ++m)
                    if (member(m)) stage[(pe0 + m) * tile_vecs + ((unsigned)u << lane_shift) + i] =
                        stream_load<NTL>(base + (uint64_t)(pe0 + m) * pe_stride + src_off + 16 * v);
            }
        }
        __syncthreads();
        // a thread folds one 4-byte word of the tile at a time - one element of 4 or 8 bytes, or the 2 or 4
        // narrower elements that share the word, each folded on its own in member order - so that a tile of
        // 1- or 2-byte elements costs as many LDS instructions as one of 4-byte elements
        for (unsigned w = threadIdx.x; w < tile_words; w += blockDim.x) {
            typedef nvshmemi_amd_fold_form<T, OP> form;
            const word_t first = stage_w[w];
            typename form::acc_t acc[EPW];
#pragma unroll
            for (int j = 0; j < EPW; ++j) acc[j] = form::lift(first.e[j]);
            if (NPES) {
#pragma unroll
                for (int p = 1; p < NPES; ++p) {
                    const word_t x = stage_w[(size_t)p * tile_words + w];
#pragma unroll
                    for (int j = 0; j < EPW; ++j) acc[j] = form::step(p, acc[j], x.e[j]);
                }
            } else {
                // eight members' values fetched from LDS before they are folded, in member order
                int p = 1;
                for (; p + 8 <= npes; p += 8) {
                    word_t x[8];
#pragma unroll
                    for (int k = 0; k < 8; ++k) x[k] = stage_w[(size_t)(p + k) * tile_words + w];
#pragma unroll
                    for (int k = 0; k < 8; ++k)
#pragma unroll
                        for (int j = 0; j < EPW; ++j) acc[j] = form::step(p + k, acc[j], x[k].e[j]);
                }
                for (; p < npes; ++p) {
                    const word_t x = stage_w[(size_t)p * tile_words + w];
#pragma unroll
                    for (int j = 0; j < EPW; ++j) acc[j] = form::step(p, acc[j], x.e[j]);
                }
            }
            word_t out;
#pragma unroll
            for (int j = 0; j < EPW; ++j) out.e[j] = form::lower(acc[j]);
            result_w[w] = out;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < VPT; ++u) {
            const uint64_t v = v0 + ((uint64_t)u << lane_shift);
            const nvshmemi_v4u r = result[((unsigned)u << lane_shift) + i];
            if (v < nvec) {
#pragma unroll
                for (int m = 0; m < MPW; ++m)
                    if (member(m)) stream_store<NVSHMEM_AMD_STORE_REDUCE>(base + (uint64_t)(pe0 + m) * pe_stride + dst_off + 16 * v, r);
            }
        }
    }
    // elements behind the last full vector
    const uint64_t done = nvec * VEC;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid < nelems - done) {
        const uint64_t k = done + gid;
        const T *s = reinterpret_cast<const T *>(base + src_off);
        T *d = reinterpret_cast<T *>(base + dst_off);
        const uint64_t es = pe_stride / sizeof(T);
        T acc = s[k];
        for (int p = 1; p < npes; ++p) acc = nvshmemi_amd_fold_step<T, OP>(p, acc, s[(uint64_t)p * es + k]);
        for (int p = 0; p < npes; ++p) d[(uint64_t)p * es + k] = acc;
    }
}

// Allreduce without LDS, for teams the LDS-staged kernel serves badly (more than 16 members: its block
// of 1024 threads leaves 32 or 16 lanes per member, i.e. 512 or 256 byte accesses): a block is ONE
// wavefront, lane i loads vector i of a 1 KiB piece from every member, eight loads in flight at a time,
// folds in member order and stores the result to every member.
// NPES > 0 fixes the team size at compile time (loads, fold and stores fully unrolled).
// ROOT_ONLY: the result goes to member 0's destination only (the first half of the two-step allreduce of large teams).
template <typename T, int OP, int NPES, bool NTL, bool ROOT_ONLY = false>
__global__ __launch_bounds__(64) void reduce_gather_kernel(char *base, uint64_t slice_bytes,
                                                           const nvshmemi_amd_team_view_t *groups,
                                                           uint64_t dst_off, uint64_t src_off, uint64_t nelems) {
    constexpr int VEC = 16 / sizeof(T);
    constexpr int kBatch = 8;
    constexpr int kBatches = NPES ? (NPES + kBatch - 1) / kBatch : 1, kStores = NPES ? NPES : 1;  // unroll counts
    union pack_t {
        nvshmemi_v4u v;
        T e[VEC];
    };
    const nvshmemi_amd_team_view_t g = groups[blockIdx.z];
    const int npes = NPES ? NPES : g.size;
    base += (uint64_t)g.start * slice_bytes;
    const uint64_t pe_stride = (uint64_t)g.stride * slice_bytes;
    const uint64_t nvec = nelems / VEC;
    const uint64_t lead = ((uint64_t)(uintptr_t)(base + dst_off) >> 4) & 63;
    const uint64_t v = (uint64_t)blockIdx.x * 64 + threadIdx.x - lead;
    if (v < nvec) {
        const char *src = base + src_off + 16 * v;
        pack_t acc;
#pragma unroll kBatches
        for (int p0 = 0; p0 < npes; p0 += kBatch) {
            pack_t x[kBatch];
#pragma unroll
            for (int k = 0; k < kBatch; ++k)
                if (p0 + k < npes) x[k].v = stream_load<NTL>(src + (uint64_t)(p0 + k) * pe_stride);
#pragma unroll
            for (int k = 0; k < kBatch; ++k)
                if (p0 + k < npes) {
                    if (p0 + k == 0) {
                        acc = x[0];
                    } else {
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            acc.e[j] = nvshmemi_amd_fold_step<T, OP>(p0 + k, acc.e[j], x[k].e[j]);
                    }
                }
        }
        char *dst = base + dst_off + 16 * v;
        if (ROOT_ONLY) {
            stream_store<NVSHMEM_AMD_STORE_REDUCESCATTER>(dst, acc.v);
        } else {
#pragma unroll kStores
            for (int p = 0; p < npes; ++p) stream_store<NVSHMEM_AMD_STORE_REDUCE>(dst + (uint64_t)p * pe_stride, acc.v);
        }
    }
    // elements behind the last full vector
    const uint64_t done = nvec * VEC;
    const uint64_t gid = (uint64_t)blockIdx.x * 64 + threadIdx.x;
    if (gid < nelems - done) {
        const uint64_t k = done + gid;
        const T *s = reinterpret_cast<const T *>(base + src_off);
        T *d = reinterpret_cast<T *>(base + dst_off);
        const uint64_t es = pe_stride / sizeof(T);
        T acc = s[k];
        for (int p = 1; p < npes; ++p) acc = nvshmemi_amd_fold_step<T, OP>(p, acc, s[(uint64_t)p * es + k]);
        for (int p = 0; p < (ROOT_ONLY ? 1 : npes); ++p) d[(uint64_t)p * es + k] = acc;
    }
}

// reducescatter without LDS: a block is ONE wavefront, lane i loads vector i of a 1 KiB piece of block q
// (blockIdx.y) from every member - eight independent loads in flight per lane at a time - folds them in
// member order in registers and stores one vector into member q's destination.  The work is nearly all
// loads, and for loads this shape beats the LDS-staged tile of the allreduce: 6.3 against 5.9 TB/s for
// 8 members with 256 MiB of source each, 5.9 against 3.7 TB/s for 16 members.  NPES > 0 fixes the team
// size at compile time; NPES == 0 reads it from the team.
template <typename T, int OP, int NPES, bool NTL>
__global__ __launch_bounds__(64) void reducescatter_gather_kernel(char *base, uint64_t slice_bytes,
                                                                  const nvshmemi_amd_team_view_t *groups,
                                                                  uint64_t dst_off, uint64_t src_off,
                                                                  uint64_t nelems) {
    constexpr int VEC = 16 / sizeof(T);
    constexpr int kBatch = 8;  // loads in flight per lane
    union pack_t {
        nvshmemi_v4u v;
        T e[VEC];
    };
    const nvshmemi_amd_team_view_t g = groups[blockIdx.z];
    const int npes = NPES ? NPES : g.size;
    if ((int)blockIdx.y >= npes) return;
    base += (uint64_t)g.start * slice_bytes;
    const uint64_t pe_stride = (uint64_t)g.stride * slice_bytes;
    const uint64_t nvec = nelems / VEC;
    src_off += (uint64_t)blockIdx.y * nelems * sizeof(T);
    // pieces are cut on absolute 1 KiB boundaries of the source: `lead` slots of piece 0 lie in front
    const uint64_t lead = ((uint64_t)(uintptr_t)(base + src_off) >> 4) & 63;
    const uint64_t v = (uint64_t)blockIdx.x * 64 + threadIdx.x - lead;
    if (v >= nvec) return;  // also the slots in front of the block (wrapped)
    const char *src = base + src_off + 16 * v;
    pack_t acc;
    for (int p0 = 0; p0 < npes; p0 += kBatch) {
        pack_t x[kBatch];
#pragma unroll
        for (int k = 0; k < kBatch; ++k)
            if (p0 + k < npes) x[k].v = stream_load<NTL>(src + (uint64_t)(p0 + k) * pe_stride);
#pragma unroll
        for (int k = 0; k < kBatch; ++k)
            if (p0 + k < npes) {
                if (p0 + k == 0) {
                    acc = x[0];
                } else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc.e[j] = nvshmemi_amd_reduce_op<T, OP>(acc.e[j], x[k].e[j]);
                }
            }
    }
    stream_store<NVSHMEM_AMD_STORE_REDUCESCATTER>(base + (uint64_t)blockIdx.y * pe_stride + dst_off + 16 * v, acc.v);
}

// Element-at-a-time variant for buffers that are not 16-byte aligned.
template <typename T, int OP, bool SCATTER = false>
__global__ __launch_bounds__(kThreads) void reduce_scalar_kernel(char *base, uint64_t slice_bytes,
                                                                 const nvshmemi_amd_team_view_t *groups,
                                                                 uint64_t dst_off, uint64_t src_off,
                                                                 uint64_t nelems) {
    const nvshmemi_amd_team_view_t g = groups[blockIdx.z];
    const int npes = g.size;
    if (SCATTER && (int)blockIdx.y >= npes) return;
    base += (uint64_t)g.start * slice_bytes;
    const uint64_t gsz = (uint64_t)gridDim.x * kThreads;
    const uint64_t es = ((uint64_t)g.stride * slice_bytes) / sizeof(T);
    const T *s = reinterpret_cast<const T *>(base + src_off) + (SCATTER ? (uint64_t)blockIdx.y * nelems : 0);
    T *d = reinterpret_cast<T *>(base + dst_off) + (SCATTER ? (uint64_t)blockIdx.y * es : 0);
    for (uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x; i < nelems; i += gsz) {
        T acc = s[i];
        for (int pe = 1; pe < npes; ++pe) acc = fold_next<T, OP, SCATTER>(pe, acc, s[(uint64_t)pe * es + i]);
        if (SCATTER) d[i] = acc;
        else for (int pe = 0; pe < npes; ++pe) d[(uint64_t)pe * es + i] = acc;
    }
}

#ifndef NVSHMEM_AMD_STORE_FCOLLECT_CHUNKED
#define NVSHMEM_AMD_STORE_FCOLLECT_CHUNKED kStoreThroughStream /* +2 % over nt */
#endif
#ifndef NVSHMEM_AMD_STORE_BROADCAST_CHUNKED
#define NVSHMEM_AMD_STORE_BROADCAST_CHUNKED kStoreStream /* +2.5 % over sc1 nt */
#endif

// Chunked sharing, the form fcollect and broadcast of sources beyond the Infinity Cache take: a wavefront stores
// its piece to two destinations, and the grid walks a chunk of tiles once per pair of destinations before it moves
// on (segment_copy_kernel, chunk_shift).  A write-dominated kernel is bound by how the memory system takes its
// writes, and that favours few write fronts: a write-only stream runs at 6.9 TB/s as ONE front sweeping memory,
// 5.7-6.2 as 64 fronts, 4.6-5.3 as 256.  With every block storing to all 8 or 16 destinations the blocks in flight
// feed 8 or 16 fronts of a few KiB each; chunked, they feed a few fronts of 2-4 MiB.  Measured (random data, 16 x
// 32 MiB fcollect / 512 MiB broadcast to 8): fcollect 5.85 -> 6.30 TB/s, broadcast 6.07 -> 6.48; the chunk that
// measured best makes chunk x groups = 16384 blocks, twice what the GPU holds at a time (fcollect: 2^11 tiles x
// 8 pairs; broadcast: 2^12 x 4; half or double that chunk loses 1-12 %), one destination per wavefront 20 %.
// Forms with at most four destinations per wavefront whose sharers are neighbouring blocks, or the wavefronts of
// one block, measured 5.85 / 6.03 TB/s on the same two workloads.  Cache-resident sources keep one wavefront per
// piece storing to every member: a split costs them up to 9 %.
#ifndef NVSHMEM_AMD_CHUNKED_REPLICAS_PER_WAVE
#define NVSHMEM_AMD_CHUNKED_REPLICAS_PER_WAVE 2
#endif
#ifndef NVSHMEM_AMD_CHUNK_CYCLE_SHIFT /* log2 of chunk tiles x destination groups */
#define NVSHMEM_AMD_CHUNK_CYCLE_SHIFT 14
#endif
// Groups of the chunked form: the largest power of two that leaves every group at least
// NVSHMEM_AMD_CHUNKED_REPLICAS_PER_WAVE destinations (16 members: 8 groups of 2; 24: 8 of 3; 5: 2 groups of 3 and 2),
// so that no group is empty.
static uint32_t chunked_part_shift(int max_size) {
    uint32_t shift = 0;
    while ((max_size >> (shift + 1)) >= NVSHMEM_AMD_CHUNKED_REPLICAS_PER_WAVE) ++shift;
    return shift;
}
static uint32_t chunk_shift_for(uint32_t part_shift) {
    const uint32_t cycle = NVSHMEM_AMD_CHUNK_CYCLE_SHIFT;
    return cycle > part_shift + 8 ? cycle - part_shift : 8;   // at least 256 tiles (a multiple of the 8 XCDs) per chunk
}

// members of all teams of the handle together
static uint64_t total_members(const TeamLaunch &tl) {
    // sizes lie between min and max; the exact sum only matters for the cache policy threshold
    return (uint64_t)tl.ngroups * (uint64_t)tl.max_size;
}

// Launches the broadcast kernel: member `root`'s [soff, +bytes) to every member's [doff, +bytes).
static int launch_broadcast(Runtime &rt, const TeamLaunch &tl, uint64_t doff, uint64_t soff, uint64_t bytes, int root,
                            hipStream_t stream, bool force_chunked = false) {
    // The chunked form from Runtime::chunked_copy_bytes (128 MiB) on: measured level with the plain form at
    // 64 MiB and 3-5 % ahead from 128 MiB for 4 and 8 members (teams of fewer than four members have one group
    // of destinations and keep the plain form).  A source that cannot stay in the Infinity Cache is streamed.
    const bool big_source = bytes * (uint64_t)tl.ngroups > rt.cacheable_source_bytes;
    const bool chunked = force_chunked || bytes * (uint64_t)tl.ngroups >= rt.chunked_copy_bytes;
    const uint32_t part_shift = chunked ? chunked_part_shift(tl.max_size) : 0;
    const uint32_t chunk_shift = part_shift ? chunk_shift_for(part_shift) : 0;
    uint64_t tiles = (bytes / 16 + 64 + kCopyThreads - 1) / kCopyThreads + 1;
    tiles = ((tiles + (1ull << chunk_shift) - 1) >> chunk_shift << chunk_shift) << part_shift;  // whole chunks
    if (tiles > 0x7fffffffull) {
        set_error("broadcast: message too large");
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    const dim3 grid((unsigned)tiles, 1, (unsigned)tl.ngroups), block(kCopyThreads);
    // blocks that share a piece re-read it from the cache, so the loads stay cacheable then
#define NVSHMEM_AMD_LAUNCH_BROADCAST(NTL, STORE)                                                      \
    hipLaunchKernelGGL((segment_copy_kernel<kModeBroadcast, 1, NTL, STORE>), grid, block, 0, stream,    \
                       rt.base, rt.heap_size, tl.groups, tl.max_size, doff, soff, (uint64_t)bytes, root, \
                       part_shift, chunk_shift)
    if (chunk_shift != 0) NVSHMEM_AMD_LAUNCH_BROADCAST(false, NVSHMEM_AMD_STORE_BROADCAST_CHUNKED);
    else if (big_source) NVSHMEM_AMD_LAUNCH_BROADCAST(true, NVSHMEM_AMD_STORE_REPLICATE);
    else NVSHMEM_AMD_LAUNCH_BROADCAST(false, NVSHMEM_AMD_STORE_REPLICATE);
#undef NVSHMEM_AMD_LAUNCH_BROADCAST
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("broadcast: kernel launch failed: %s", hipGetErrorString(e));
        return NVSHMEMX_ERROR_INTERNAL;
    }
    return 0;
}

template <typename T, int OP>
void launch_reduce(Runtime &rt, const TeamLaunch &tl, uint64_t dst_off, uint64_t src_off,
                   uint64_t nelems, hipStream_t stream) {
    const bool vector_ok = ((dst_off | src_off) & 15) == 0;
    const unsigned ngroups = (unsigned)tl.ngroups;
    // Which vector kernel.  From Runtime::lds_reduce_bytes of sources in all (64 MiB; a quarter
    // of that for teams of 17 to 32 members, four times for larger ones) the LDS-staged
    // kernel wins for every team of 3 to 64 members; below that, and for 2 members, the gather kernel does.
    // fp32 sum on a stream, LDS-staged / gather in TB/s, sources of 32 MiB | 64 MiB | 128 MiB in all: 4 members
    // 7.3 / 8.4 | 7.6 / 7.4 | 8.3 / 8.1, 8 members 7.8 / 8.3 | 7.8 / 6.9 | 8.5 / 7.7, 16 members 7.0 / 8.3 |
    // 7.6 / 6.6 | 8.3 / 7.6; 32 members lead with the LDS kernel from 16 MiB on (7.3 / 5.3), 48 and 64 members
    // with the gather kernel up to 128-192 MiB (5.9 / 6.8).  Beyond the cache,
    // measured with random fp32 data and write-through stores, LDS-staged against gather, TB/s at
    // 512 MiB / 2 GiB of sources: 4 members 6.54 / 6.55 against 6.19 / 6.24, 6 members 6.37 / 6.44
    // against 5.89 / 5.58, 8 members 6.46 / 6.53 against 6.03 / 6.09, 12 members 6.28 / 6.28 against
    // 5.73 / 5.83, 16 members 6.21 / 6.12 against 5.44 / 5.57, 32 members 6.17 / 6.10 against 5.22 / 5.49,
    // 64 members 5.64 / 5.64 against 5.15 / 5.26.  A wavefront of the LDS kernel serves one member
    // for the compile-time sizes 8 and 16, two members up to 32 and four beyond: one load and one store
    // per lane measured best where the block stays within 16 wavefronts, and wavefronts of fewer than
    // 64 lanes per member (512- or 256-byte accesses) lost 7-22 % against the gather kernel.  The
    // compile-time team size is worth 6 % at 32 members (6.17 against 5.82), nothing at 64.
    const uint64_t total_bytes = total_members(tl) * nelems * sizeof(T);
    const int fixed_size = tl.min_size == tl.max_size ? tl.max_size : 0;
    const bool stream_source = total_bytes > rt.cacheable_source_bytes;
    // (in bytes whatever the element type: fp32, bf16 and int64 cross over at the same 64 MiB on 8 and 16 members)
    const uint64_t lds_from_bytes = tl.max_size > 32   ? rt.lds_reduce_bytes * 4
                                    : tl.max_size > 16 ? rt.lds_reduce_bytes / 4
                                                       : rt.lds_reduce_bytes;
    // mpw: members per wavefront of the LDS-staged kernel; ct_size: a compile-time team size, if any
    int mpw = 0, ct_size = 0;
    constexpr int kNarrowMpw = sizeof(T) <= 2 ? NVSHMEM_AMD_REDUCE_NARROW_MPW : NVSHMEM_AMD_REDUCE_WIDE_MPW;
    if (fixed_size == 8 || fixed_size == 16) ct_size = fixed_size, mpw = kNarrowMpw;
    else if (fixed_size == 32) ct_size = 32, mpw = 2;
    else if (tl.max_size >= 3 && tl.max_size <= 32) mpw = 2;
    else if (tl.max_size > 32 && tl.max_size <= 64) mpw = 4;
    // Two-step allreduce of large teams: fold into member 0's destination (n loads and ONE store per vector, the
    // shape of the reducescatter), then broadcast that in the chunked form.  It moves 2 n + 2 units where the fused
    // kernel moves 2 n, but every block of the fused kernel feeds n write fronts of 1 KiB pieces, and its fold
    // serialises n steps between two barriers.  fp32 sum, TB/s, fused / two-step at 512 MiB and 2 GiB of sources in
    // all: 12 members 6.41 / 6.18 and 6.28 / 6.29, 16: 6.26 / 6.19 and 6.02 / 6.41, 24: 5.84 / 5.71 and 5.69 / 6.23,
    // 32: 6.09 / 6.09 and 6.09 / 6.51, 48: 5.68 / 5.78 and 5.57 / 6.25, 64: 5.55 / 5.97 and 5.59 / 6.56.  So: from
    // Runtime::two_step_reduce_members (16) members on when the sources hold two_step_reduce_bytes (512 MiB: 16 members 6.2 against 6.0 TB/s fused there, 32 members 6.3 against 5.8) or more,
    // and from three times that many members whatever the size.
    if (vector_ok && rt.two_step_reduce_members && tl.min_size >= (int)rt.two_step_reduce_members &&
        (total_bytes >= rt.two_step_reduce_bytes || tl.min_size >= 3 * (int)rt.two_step_reduce_members) &&
        total_bytes >= lds_from_bytes) {
        const uint64_t nvec = nelems / (16 / sizeof(T));
        uint64_t blocks = (nvec + 63 + 63) / 64;
        if (blocks <= 0x7fffffffull) {
            const dim3 grid((unsigned)blocks, 1, ngroups);
            if (stream_source)
                hipLaunchKernelGGL((reduce_gather_kernel<T, OP, 0, true, true>), grid, dim3(64), 0, stream, rt.base,
                                   rt.heap_size, tl.groups, dst_off, src_off, nelems);
            else
                hipLaunchKernelGGL((reduce_gather_kernel<T, OP, 0, false, true>), grid, dim3(64), 0, stream, rt.base,
                                   rt.heap_size, tl.groups, dst_off, src_off, nelems);
            (void)launch_broadcast(rt, tl, dst_off, dst_off, nelems * sizeof(T), 0, stream, true);
            return;
        }
    }
    if (vector_ok && mpw && total_bytes >= lds_from_bytes) {
        const uint32_t lane_shift = 6;
        const unsigned threads = (unsigned)((tl.max_size + mpw - 1) / mpw) << lane_shift;
        const uint64_t nvec = nelems / (16 / sizeof(T));
        // A tile of two vectors per thread halves the barriers per byte: worth 5 % for 16-bit elements with one
        // member per wavefront (bf16 sum at 8 x 128 MiB 5.83 -> 6.14 TB/s), less than the two members per
        // wavefront they now use with one vector; it costs 4-byte and 8-byte elements 3-4 %.
        constexpr int kVptNarrow = sizeof(T) <= 2 ? NVSHMEM_AMD_REDUCE_VPT_NARROW : NVSHMEM_AMD_REDUCE_VPT;
        const int vpt = (ct_size == 8 || ct_size == 16) ? kVptNarrow : NVSHMEM_AMD_REDUCE_VPT;
        const uint64_t tile_vecs = (uint64_t)vpt << lane_shift;
        uint64_t blocks = (nvec + (1u << lane_shift) + tile_vecs - 1) / tile_vecs;  // room for the lead-in
        if (blocks > 0x7fffffffull) blocks = 0x7fffffffull;  // the tile loop covers the rest
        const size_t lds = ((size_t)tl.max_size + 1) * 16 * tile_vecs;
        const dim3 grid((unsigned)blocks, 1, ngroups);
#define NVSHMEM_AMD_LAUNCH_REDUCE(N, MPW) NVSHMEM_AMD_LAUNCH_REDUCE_V(N, MPW, NVSHMEM_AMD_REDUCE_VPT)
#define NVSHMEM_AMD_LAUNCH_REDUCE_V(N, MPW, VPT)                                                  \
    do {                                                                                          \
        if (stream_source)                                                                        \
            hipLaunchKernelGGL((reduce_vector_kernel<T, OP, N, true, VPT, MPW>), grid, dim3(threads), lds,  \
                               stream, rt.base, rt.heap_size, tl.groups, dst_off,    \
                               src_off, nelems);                                                  \
        else                                                                                      \
            hipLaunchKernelGGL((reduce_vector_kernel<T, OP, N, false, VPT, MPW>), grid, dim3(threads), lds, \
                               stream, rt.base, rt.heap_size, tl.groups, dst_off,    \
                               src_off, nelems);                                                  \
    } while (0)
        if (ct_size == 8) NVSHMEM_AMD_LAUNCH_REDUCE_V(8, kNarrowMpw, kVptNarrow);
        else if (ct_size == 16) NVSHMEM_AMD_LAUNCH_REDUCE_V(16, kNarrowMpw, kVptNarrow);
        else if (ct_size == 32) NVSHMEM_AMD_LAUNCH_REDUCE(32, 2);
        else if (mpw == 2) NVSHMEM_AMD_LAUNCH_REDUCE(0, 2);
        else NVSHMEM_AMD_LAUNCH_REDUCE(0, 4);
#undef NVSHMEM_AMD_LAUNCH_REDUCE
#undef NVSHMEM_AMD_LAUNCH_REDUCE_V
    } else if (vector_ok) {
        const uint64_t nvec = nelems / (16 / sizeof(T));
        uint64_t blocks = (nvec + 63 + 63) / 64;  // room for the lead-in; at least one block for the tail
        if (blocks > 0x7fffffffull) {
            set_error("reduce: message too large");
            return;
        }
        const dim3 grid((unsigned)blocks, 1, ngroups);
#define NVSHMEM_AMD_LAUNCH_GATHER_REDUCE(N)                                                            \
    do {                                                                                               \
        if (stream_source)                                                                             \
            hipLaunchKernelGGL((reduce_gather_kernel<T, OP, N, true>), grid, dim3(64), 0, stream, rt.base, \
                               rt.heap_size, tl.groups, dst_off, src_off, nelems);                    \
        else                                                                                           \
            hipLaunchKernelGGL((reduce_gather_kernel<T, OP, N, false>), grid, dim3(64), 0, stream, rt.base, \
                               rt.heap_size, tl.groups, dst_off, src_off, nelems);                    \
    } while (0)
        // (sixteen members unrolled measured slower than the loop: 5.2 against 5.4 TB/s)
        if (fixed_size == 4) NVSHMEM_AMD_LAUNCH_GATHER_REDUCE(4);
        else if (fixed_size == 8) NVSHMEM_AMD_LAUNCH_GATHER_REDUCE(8);
        else NVSHMEM_AMD_LAUNCH_GATHER_REDUCE(0);
#undef NVSHMEM_AMD_LAUNCH_GATHER_REDUCE
    } else {
        uint64_t blocks = (nelems + kThreads - 1) / kThreads;
        const uint64_t cap = (uint64_t)rt.num_cus * 64 / ngroups + 1;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL((reduce_scalar_kernel<T, OP>), dim3((unsigned)blocks, 1, ngroups),
                           dim3(kThreads), 0, stream, rt.base, rt.heap_size, tl.groups, dst_off,
                           src_off, nelems);
    }
}

// reducescatter: grid.y = destination member; nelems is the element count of one PE's result
template <typename T, int OP>
void launch_reducescatter(Runtime &rt, const TeamLaunch &tl, uint64_t dst_off, uint64_t src_off,
                          uint64_t nelems, hipStream_t stream) {
    const bool vector_ok = ((dst_off | src_off | (nelems * sizeof(T))) & 15) == 0;
    const unsigned ngroups = (unsigned)tl.ngroups;
    if (vector_ok) {
        const uint64_t nvec = nelems / (16 / sizeof(T));
        uint64_t blocks = (nvec + 63 + 63) / 64;  // room for the lead-in
        if (blocks > 0x7fffffffull) {
            set_error("reducescatter: message too large");
            return;
        }
        const dim3 grid((unsigned)blocks, (unsigned)tl.max_size, ngroups);
        const bool stream_source =
            total_members(tl) * tl.max_size * nelems * sizeof(T) > rt.cacheable_source_bytes;
#define NVSHMEM_AMD_LAUNCH_GATHER(N, NTL)                                                         \
    hipLaunchKernelGGL((reducescatter_gather_kernel<T, OP, N, NTL>), grid, dim3(64), 0, stream,   \
                       rt.base, rt.heap_size, tl.groups, dst_off, src_off, nelems)
        if (tl.min_size == 8 && tl.max_size == 8) {
            if (stream_source) NVSHMEM_AMD_LAUNCH_GATHER(8, true);
            else NVSHMEM_AMD_LAUNCH_GATHER(8, false);
        } else {
            if (stream_source) NVSHMEM_AMD_LAUNCH_GATHER(0, true);
            else NVSHMEM_AMD_LAUNCH_GATHER(0, false);
        }
#undef NVSHMEM_AMD_LAUNCH_GATHER
    } else {
        uint64_t blocks = (nelems + kThreads - 1) / kThreads;
        const uint64_t cap = (uint64_t)rt.num_cus * 64 / ((uint64_t)tl.max_size * ngroups) + 1;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL((reduce_scalar_kernel<T, OP, true>),
                           dim3((unsigned)blocks, (unsigned)tl.max_size, ngroups), dim3(kThreads), 0,
                           stream, rt.base, rt.heap_size, tl.groups, dst_off, src_off, nelems);
    }
}

typedef void (*reduce_launcher_t)(Runtime &, const TeamLaunch &, uint64_t, uint64_t, uint64_t,
                                  hipStream_t);

template <typename T, bool SCATTER>
reduce_launcher_t pick_arith(int op) {
#define NVSHMEM_AMD_PICK(OP) \
    case NVSHMEMI_OP_##OP: return SCATTER ? launch_reducescatter<T, NVSHMEMI_OP_##OP> : launch_reduce<T, NVSHMEMI_OP_##OP>
    switch (op) {
        NVSHMEM_AMD_PICK(min);
        NVSHMEM_AMD_PICK(max);
        NVSHMEM_AMD_PICK(sum);
        NVSHMEM_AMD_PICK(prod);
        default: return nullptr;
    }
}
template <typename T, bool SCATTER>
reduce_launcher_t pick_integer(int op) {
    switch (op) {
        NVSHMEM_AMD_PICK(and);
        NVSHMEM_AMD_PICK(or);
        NVSHMEM_AMD_PICK(xor);
        default: return pick_arith<T, SCATTER>(op);
    }
#undef NVSHMEM_AMD_PICK
}

template <bool SCATTER>
reduce_launcher_t pick_reduce(int dtype, int op) {
    switch (dtype) {
        case NVSHMEMI_DT_i8: return pick_integer<int8_t, SCATTER>(op);
        case NVSHMEMI_DT_i16: return pick_integer<int16_t, SCATTER>(op);
        case NVSHMEMI_DT_i32: return pick_integer<int32_t, SCATTER>(op);
        case NVSHMEMI_DT_i64: return pick_integer<int64_t, SCATTER>(op);
        case NVSHMEMI_DT_u8: return pick_integer<uint8_t, SCATTER>(op);
        case NVSHMEMI_DT_u16: return pick_integer<uint16_t, SCATTER>(op);
        case NVSHMEMI_DT_u32: return pick_integer<uint32_t, SCATTER>(op);
        case NVSHMEMI_DT_u64: return pick_integer<uint64_t, SCATTER>(op);
        case NVSHMEMI_DT_f16: return pick_arith<__half, SCATTER>(op);
        case NVSHMEMI_DT_bf16: return pick_arith<__hip_bfloat16, SCATTER>(op);
        case NVSHMEMI_DT_f32: return pick_arith<float, SCATTER>(op);
        case NVSHMEMI_DT_f64: return pick_arith<double, SCATTER>(op);
        default: return nullptr;
    }
}

const size_t kDtypeSize[NVSHMEMI_DT_COUNT] = {1, 2, 4, 8, 1, 2, 4, 8, 2, 2, 4, 8};

}  // namespace

int reduce_on_stream(int dtype, int op, nvshmem_team_t team, void *dest, const void *src,
                     size_t nreduce, hipStream_t stream) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    TeamLaunch tl;
    if (!resolve_team(rt, "reduce", team, &tl)) return NVSHMEMX_ERROR_INVALID_VALUE;
    reduce_launcher_t fn = pick_reduce<false>(dtype, op);
    if (!fn) {
        set_error("reduce: operator %d is not defined for element kind %d", op, dtype);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    if (nreduce == 0) return 0;
    const size_t es = kDtypeSize[dtype];
    uint64_t doff = 0, soff = 0;
    if (nreduce > rt.heap_size / es) {
        set_error("reduce: %zu elements of %zu bytes leave the PE's heap slice", nreduce, es);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    if (!check_symmetric_range(rt, "reduce dest", dest, nreduce * es, &doff) ||
        !check_symmetric_range(rt, "reduce source", src, nreduce * es, &soff))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if ((doff % es) || (soff % es)) {
        set_error("reduce: buffers must be aligned to the element size");
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    if (doff != soff && doff < soff + nreduce * es && soff < doff + nreduce * es) {
        set_error("reduce: dest and source overlap without being identical");
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    fn(rt, tl, doff, soff, nreduce, stream);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("reduce: kernel launch failed: %s", hipGetErrorString(e));
        return NVSHMEMX_ERROR_INTERNAL;
    }
    return 0;
}

int reducescatter_on_stream(int dtype, int op, nvshmem_team_t team, void *dest, const void *src,
                            size_t nreduce, hipStream_t stream) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    TeamLaunch tl;
    if (!resolve_team(rt, "reducescatter", team, &tl)) return NVSHMEMX_ERROR_INVALID_VALUE;
    reduce_launcher_t fn = pick_reduce<true>(dtype, op);
    if (!fn) {
        set_error("reducescatter: operator %d is not defined for element kind %d", op, dtype);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    if (nreduce == 0) return 0;
    const size_t es = kDtypeSize[dtype];
    const uint64_t n = (uint64_t)tl.max_size;
    if (nreduce > rt.heap_size / es / n) {
        set_error("reducescatter: %zu elements of %zu bytes x %d PEs leave the PE's heap slice",
                  nreduce, es, tl.max_size);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    uint64_t doff = 0, soff = 0;
    if (!check_symmetric_range(rt, "reducescatter dest", dest, nreduce * es, &doff) ||
        !check_symmetric_range(rt, "reducescatter source", src, nreduce * es * n, &soff))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if ((doff % es) || (soff % es)) {
        set_error("reducescatter: buffers must be aligned to the element size");
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    // PE q writes dest while other PEs' blocks of the source at the same offsets are still read
    if (doff < soff + nreduce * es * n && soff < doff + nreduce * es) {
        set_error("reducescatter: dest and source overlap");
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    fn(rt, tl, doff, soff, nreduce, stream);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("reducescatter: kernel launch failed: %s", hipGetErrorString(e));
        return NVSHMEMX_ERROR_INTERNAL;
    }
    return 0;
}

int broadcast_on_stream(nvshmem_team_t team, void *dest, const void *src, size_t bytes, int root,
                        hipStream_t stream) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    TeamLaunch tl;
    if (!resolve_team(rt, "broadcast", team, &tl)) return NVSHMEMX_ERROR_INVALID_VALUE;
    if (root < 0 || root >= tl.min_size) {
        set_error("broadcast: root %d is not a PE of the team (0..%d)", root, tl.min_size - 1);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    if (bytes == 0) return 0;
    uint64_t doff = 0, soff = 0;
    if (!check_symmetric_range(rt, "broadcast dest", dest, bytes, &doff) ||
        !check_symmetric_range(rt, "broadcast source", src, bytes, &soff))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    // identical buffers are the in-place form (the root keeps its data); a partial overlap would
    // let the root's destination clobber source bytes that are still to be read
    if (doff != soff && doff < soff + bytes && soff < doff + bytes) {
        set_error("broadcast: dest and source overlap without being identical");
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    return launch_broadcast(rt, tl, doff, soff, bytes, root, stream);
}

static int segment_collective(int mode, const char *what, nvshmem_team_t team, void *dest,
                              const void *src, size_t seg_bytes, hipStream_t stream) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    TeamLaunch tl;
    if (!resolve_team(rt, what, team, &tl)) return NVSHMEMX_ERROR_INVALID_VALUE;
    if (seg_bytes == 0) return 0;
    const uint64_t n = (uint64_t)tl.max_size;
    if (seg_bytes > rt.heap_size / n) {
        set_error("%s: %zu bytes x %d PEs does not fit a PE's heap slice", what, seg_bytes, tl.max_size);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    const uint64_t src_bytes = mode == kModeFcollect ? seg_bytes : seg_bytes * n;
    uint64_t doff = 0, soff = 0;
    if (!check_symmetric_range(rt, what, dest, seg_bytes * n, &doff) ||
        !check_symmetric_range(rt, what, src, src_bytes, &soff))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if (doff < soff + src_bytes && soff < doff + seg_bytes * n) {
        set_error("%s: dest and source overlap", what);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    const uint64_t tile_vectors = (uint64_t)kCopyThreads * (mode == kModeFcollect ? NVSHMEM_AMD_FCOLLECT_UNROLL
                                                                              : NVSHMEM_AMD_ALLTOALL_UNROLL);
    const bool big_source = src_bytes * total_members(tl) > rt.cacheable_source_bytes;
    // An fcollect takes the chunked form when its sources hold Runtime::chunked_copy_bytes (128 MiB) or more and
    // its destinations eight times that: with the sources still in the Infinity Cache it is the n-fold larger
    // destinations that decide.  Chunked / plain in TB/s at 64 | 128 | 256 MiB of sources: 16 members 6.3 / 6.5 |
    // 7.2 / 6.6 | 7.7 / 6.5, 8 members 6.4 / 6.9 | 7.3 / 6.9 | 7.9 / 6.9, 4 members 6.7 / 7.7 | 7.7 / 8.0 | 8.4 / 8.1.
    const uint64_t all_sources = src_bytes * total_members(tl);
    const bool chunked = mode == kModeFcollect && all_sources >= rt.chunked_copy_bytes &&
                         all_sources * n >= 8 * rt.chunked_copy_bytes;
    const uint32_t part_shift = chunked ? chunked_part_shift(tl.max_size) : 0;
    const uint32_t chunk_shift = part_shift ? chunk_shift_for(part_shift) : 0;
    uint64_t tiles = (seg_bytes / 16 + 64 + tile_vectors - 1) / tile_vectors + 1;
    tiles = ((tiles + (1ull << chunk_shift) - 1) >> chunk_shift << chunk_shift) << part_shift;  // whole chunks
    const unsigned segs = mode == kModeFcollect ? (unsigned)n : (unsigned)(n * n);
    if (tiles > 0x7fffffffull) {
        set_error("%s: message too large", what);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    // blocks that share a piece re-read it from the cache, so the loads stay cacheable then
    const bool stream_source = part_shift == 0 && big_source;
    const dim3 grid((unsigned)tiles, segs, (unsigned)tl.ngroups), block(kCopyThreads);
#define NVSHMEM_AMD_LAUNCH_SEGCOPY(MODE, U, NTL, STORE)                                            \
    hipLaunchKernelGGL((segment_copy_kernel<MODE, U, NTL, STORE>), grid, block, 0, stream, rt.base, \
                       rt.heap_size, tl.groups, tl.max_size, doff, soff, (uint64_t)seg_bytes, 0,   \
                       part_shift, chunk_shift)
    if (mode == kModeFcollect) {
        if (chunk_shift != 0)
            NVSHMEM_AMD_LAUNCH_SEGCOPY(kModeFcollect, NVSHMEM_AMD_FCOLLECT_UNROLL, false, NVSHMEM_AMD_STORE_FCOLLECT_CHUNKED);
        else if (stream_source)
            NVSHMEM_AMD_LAUNCH_SEGCOPY(kModeFcollect, NVSHMEM_AMD_FCOLLECT_UNROLL, true, NVSHMEM_AMD_STORE_REPLICATE);
        else
            NVSHMEM_AMD_LAUNCH_SEGCOPY(kModeFcollect, NVSHMEM_AMD_FCOLLECT_UNROLL, false, NVSHMEM_AMD_STORE_REPLICATE);
    } else {
        if (stream_source) NVSHMEM_AMD_LAUNCH_SEGCOPY(kModeAlltoall, NVSHMEM_AMD_ALLTOALL_UNROLL, true, NVSHMEM_AMD_STORE_ALLTOALL);
        else NVSHMEM_AMD_LAUNCH_SEGCOPY(kModeAlltoall, NVSHMEM_AMD_ALLTOALL_UNROLL, false, NVSHMEM_AMD_STORE_ALLTOALL);
    }
#undef NVSHMEM_AMD_LAUNCH_SEGCOPY
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: kernel launch failed: %s", what, hipGetErrorString(e));
        return NVSHMEMX_ERROR_INTERNAL;
    }
    return 0;
}

int fcollect_on_stream(nvshmem_team_t team, void *dest, const void *src, size_t bytes,
                       hipStream_t stream) {
    return segment_collective(kModeFcollect, "fcollect", team, dest, src, bytes, stream);
}
int alltoall_on_stream(nvshmem_team_t team, void *dest, const void *src, size_t bytes,
                       hipStream_t stream) {
    return segment_collective(kModeAlltoall, "alltoall", team, dest, src, bytes, stream);
}

static int finish_blocking(int rc) {
    if (rc == 0) NVSHMEM_AMD_HIP_CHECK(hipStreamSynchronize(nullptr));
    return rc;
}

}  // namespace nvshmem_amd

using namespace nvshmem_amd;

extern "C" {

#define NVSHMEMI_DEFINE_TYPED_COLL_HOST(NAME, TYPE, TAG)                                          \
    int nvshmemx_##NAME##_alltoall_on_stream(nvshmem_team_t team, TYPE *dest, const TYPE *src,    \
                                             size_t nelems, nvshmemx_stream_t s) {                \
        return alltoall_on_stream(team, dest, src, nelems * sizeof(TYPE), (hipStream_t)s);        \
    }                                                                                             \
    int nvshmemx_##NAME##_fcollect_on_stream(nvshmem_team_t team, TYPE *dest, const TYPE *src,    \
                                             size_t nelems, nvshmemx_stream_t s) {                \
        return fcollect_on_stream(team, dest, src, nelems * sizeof(TYPE), (hipStream_t)s);        \
    }                                                                                             \
    int nvshmemx_##NAME##_broadcast_on_stream(nvshmem_team_t team, TYPE *dest, const TYPE *src,   \
                                              size_t nelems, int PE_root, nvshmemx_stream_t s) {  \
        return broadcast_on_stream(team, dest, src, nelems * sizeof(TYPE), PE_root,               \
                                   (hipStream_t)s);                                               \
    }                                                                                             \
    int nvshmem_##NAME##_broadcast(nvshmem_team_t team, TYPE *dest, const TYPE *src,              \
                                   size_t nelems, int PE_root) {                                  \
        return finish_blocking(                                                                   \
            broadcast_on_stream(team, dest, src, nelems * sizeof(TYPE), PE_root, nullptr));       \
    }                                                                                             \
    int nvshmem_##NAME##_alltoall(nvshmem_team_t team, TYPE *dest, const TYPE *src,               \
                                  size_t nelems) {                                                \
        return finish_blocking(                                                                   \
            alltoall_on_stream(team, dest, src, nelems * sizeof(TYPE), nullptr));                 \
    }                                                                                             \
    int nvshmem_##NAME##_fcollect(nvshmem_team_t team, TYPE *dest, const TYPE *src,               \
                                  size_t nelems) {                                                \
        return finish_blocking(                                                                   \
            fcollect_on_stream(team, dest, src, nelems * sizeof(TYPE), nullptr));                 \
    }
NVSHMEMI_REPT_FOR_STANDARD_RMA_TYPES(NVSHMEMI_DEFINE_TYPED_COLL_HOST)
#undef NVSHMEMI_DEFINE_TYPED_COLL_HOST

int nvshmemx_alltoallmem_on_stream(nvshmem_team_t team, void *dest, const void *src, size_t nelems,
                                   nvshmemx_stream_t stream) {
    return alltoall_on_stream(team, dest, src, nelems, (hipStream_t)stream);
}
int nvshmemx_fcollectmem_on_stream(nvshmem_team_t team, void *dest, const void *src, size_t nelems,
                                   nvshmemx_stream_t stream) {
    return fcollect_on_stream(team, dest, src, nelems, (hipStream_t)stream);
}
int nvshmemx_broadcastmem_on_stream(nvshmem_team_t team, void *dest, const void *src, size_t nelems,
                                    int PE_root, nvshmemx_stream_t stream) {
    return broadcast_on_stream(team, dest, src, nelems, PE_root, (hipStream_t)stream);
}
int nvshmem_broadcastmem(nvshmem_team_t team, void *dest, const void *src, size_t nelems,
                         int PE_root) {
    return finish_blocking(broadcast_on_stream(team, dest, src, nelems, PE_root, nullptr));
}
int nvshmem_alltoallmem(nvshmem_team_t team, void *dest, const void *src, size_t nelems) {
    return finish_blocking(alltoall_on_stream(team, dest, src, nelems, nullptr));
}
int nvshmem_fcollectmem(nvshmem_team_t team, void *dest, const void *src, size_t nelems) {
    return finish_blocking(fcollect_on_stream(team, dest, src, nelems, nullptr));
}

#define NVSHMEMI_DEFINE_TYPED_REDUCE_HOST(NAME, TYPE, TAG, OP)                                    \
    int nvshmemx_##NAME##_##OP##_reduce_on_stream(nvshmem_team_t team, TYPE *dest,                \
                                                  const TYPE *src, size_t nreduce,                \
                                                  nvshmemx_stream_t s) {                          \
        return reduce_on_stream(NVSHMEMI_DT_##TAG, NVSHMEMI_OP_##OP, team, dest, src, nreduce,    \
                                (hipStream_t)s);                                                  \
    }                                                                                             \
    int nvshmem_##NAME##_##OP##_reduce(nvshmem_team_t team, TYPE *dest, const TYPE *src,          \
                                       size_t nreduce) {                                          \
        return finish_blocking(reduce_on_stream(NVSHMEMI_DT_##TAG, NVSHMEMI_OP_##OP, team, dest,  \
                                                src, nreduce, nullptr));                          \
    }                                                                                             \
    int nvshmemx_##NAME##_##OP##_reducescatter_on_stream(nvshmem_team_t team, TYPE *dest,         \
                                                         const TYPE *src, size_t nreduce,         \
                                                         nvshmemx_stream_t s) {                   \
        return reducescatter_on_stream(NVSHMEMI_DT_##TAG, NVSHMEMI_OP_##OP, team, dest, src,      \
                                       nreduce, (hipStream_t)s);                                  \
    }                                                                                             \
    int nvshmem_##NAME##_##OP##_reducescatter(nvshmem_team_t team, TYPE *dest, const TYPE *src,   \
                                              size_t nreduce) {                                   \
        return finish_blocking(reducescatter_on_stream(NVSHMEMI_DT_##TAG, NVSHMEMI_OP_##OP, team, \
                                                       dest, src, nreduce, nullptr));             \
    }
NVSHMEMI_REPT_FOR_ALL_REDUCE_TYPES_AND_OPS(NVSHMEMI_DEFINE_TYPED_REDUCE_HOST)
#undef NVSHMEMI_DEFINE_TYPED_REDUCE_HOST

}  // extern "C"
