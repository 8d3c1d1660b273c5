// Host-launched collectives for logical PEs on one MI355X: one grid-wide kernel per call serves
// every PE of the team.
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
#include <cstdio>

#include "nvshmem.h"
#include "runtime.hpp"

namespace nvshmem_amd {
namespace {

constexpr int kThreads = 256;

// ---------------------------------------------------------------------------------------------
// Segment copy: fcollect and alltoall are sets of contiguous (source, destination) segments.
// grid.y indexes the segment, grid.x the 32 KiB tile inside it.  The destination is written with
// aligned 16-byte vectors only: block 0 of a segment copies the byte head in front of the first
// aligned destination vector and the byte tail behind the last one.
// ---------------------------------------------------------------------------------------------
constexpr int kCopyUnroll = 8;
constexpr size_t kTileVectors = (size_t)kThreads * kCopyUnroll;

enum { kModeFcollect = 0, kModeAlltoall = 1 };

template <bool SRC_ALIGNED, bool REPLICATE>
__device__ __forceinline__ void copy_tile(char *__restrict__ dst, const char *__restrict__ src,
                                          size_t nvec, uint64_t rep_stride, int nrep) {
    // nvec <= kTileVectors vectors, thread t takes t, t+256, ...
    nvshmemi_v4u v[kCopyUnroll];
    const size_t t = threadIdx.x;
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) {
        const size_t i = t + (size_t)u * kThreads;
        if (i < nvec) v[u] = nvshmemi_amd_load16<SRC_ALIGNED>(src + 16 * i);
    }
    if (REPLICATE) {
        for (int r = 0; r < nrep; ++r) {
            char *d = dst + (uint64_t)r * rep_stride;
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u) {
                const size_t i = t + (size_t)u * kThreads;
                if (i < nvec) *reinterpret_cast<nvshmemi_v4u *>(d + 16 * i) = v[u];
            }
        }
    } else {
#pragma unroll
        for (int u = 0; u < kCopyUnroll; ++u) {
            const size_t i = t + (size_t)u * kThreads;
            if (i < nvec) *reinterpret_cast<nvshmemi_v4u *>(dst + 16 * i) = v[u];
        }
    }
}

template <int MODE>
__global__ __launch_bounds__(kThreads) void segment_copy_kernel(char *base, uint32_t shift, int npes,
                                                                uint64_t dst_off, uint64_t src_off,
                                                                uint64_t seg_bytes) {
    const unsigned seg = blockIdx.y;
    const char *src;
    char *dst;
    int nrep;
    if (MODE == kModeFcollect) {
        // segment p: PE p's source -> slot p of every PE's destination
        src = base + ((uint64_t)seg << shift) + src_off;
        dst = base + dst_off + (uint64_t)seg * seg_bytes;
        nrep = npes;
    } else {
        // segment (p, q): block q of PE p's source -> slot p of PE q's destination
        const unsigned p = seg / (unsigned)npes, q = seg % (unsigned)npes;
        src = base + ((uint64_t)p << shift) + src_off + (uint64_t)q * seg_bytes;
        dst = base + ((uint64_t)q << shift) + dst_off + (uint64_t)p * seg_bytes;
        nrep = 1;
    }
    const uint64_t rep_stride = 1ull << shift;

    uint64_t head = (uint64_t)(-(uintptr_t)dst & 15);
    if (head > seg_bytes) head = seg_bytes;
    const uint64_t nvec_total = (seg_bytes - head) / 16;
    const uint64_t tail_start = head + nvec_total * 16;

    if (blockIdx.x == 0) {
        // at most 15 + 15 bytes per replica
        const uint64_t edge = head + (seg_bytes - tail_start);
        for (uint64_t e = threadIdx.x; e < edge * (uint64_t)nrep; e += kThreads) {
            const uint64_t r = e / edge, k = e % edge;
            const uint64_t pos = k < head ? k : tail_start + (k - head);
            dst[r * rep_stride + pos] = src[pos];
        }
    }
    const uint64_t first = (uint64_t)blockIdx.x * kTileVectors;
    if (first >= nvec_total) return;
    const uint64_t left = nvec_total - first;
    const size_t nvec = left < kTileVectors ? (size_t)left : kTileVectors;
    const char *s = src + head + first * 16;
    char *d = dst + head + first * 16;
    const bool aligned = (((uintptr_t)s) & 15) == 0;
    if (MODE == kModeFcollect) {
        if (aligned) copy_tile<true, true>(d, s, nvec, rep_stride, nrep);
        else copy_tile<false, true>(d, s, nvec, rep_stride, nrep);
    } else {
        if (aligned) copy_tile<true, false>(d, s, nvec, rep_stride, 1);
        else copy_tile<false, false>(d, s, nvec, rep_stride, 1);
    }
}

// ---------------------------------------------------------------------------------------------
// Fused reduce.  A lane owns 16-byte vectors of the element range; for each it loads that vector
// from every PE's source (groups of four PEs in flight, two vectors per lane), folds in PE order,
// and stores the result into every PE's destination.  An element is read by exactly one lane
// before that lane writes it, so dest == src (in place) needs no staging.
// ---------------------------------------------------------------------------------------------
constexpr int kReduceUnroll = 2;
constexpr int kPeGroup = 4;

template <typename T>
struct alignas(16) Pack {
    static constexpr int N = 16 / sizeof(T);
    T e[N];
};

template <typename T, int OP>
__global__ __launch_bounds__(kThreads) void reduce_vector_kernel(char *base, uint32_t shift, int npes,
                                                                 uint64_t dst_off, uint64_t src_off,
                                                                 uint64_t nelems) {
    typedef Pack<T> P;
    const uint64_t nvec = nelems / P::N;
    const uint64_t gsz = (uint64_t)gridDim.x * kThreads;
    const uint64_t gid = (uint64_t)blockIdx.x * kThreads + threadIdx.x;
    const uint64_t pe_stride = 1ull << shift;
    const char *src0 = base + src_off;
    char *dst0 = base + dst_off;

    for (uint64_t v0 = gid; v0 < nvec; v0 += gsz * kReduceUnroll) {
        P acc[kReduceUnroll];
        for (int g = 0; g < npes; g += kPeGroup) {
            P x[kPeGroup][kReduceUnroll];
#pragma unroll
            for (int j = 0; j < kPeGroup; ++j) {
#pragma unroll
                for (int u = 0; u < kReduceUnroll; ++u) {
                    const uint64_t v = v0 + (uint64_t)u * gsz;
                    if (g + j < npes && v < nvec)
                        x[j][u] = *reinterpret_cast<const P *>(src0 + (uint64_t)(g + j) * pe_stride + 16 * v);
                }
            }
#pragma unroll
            for (int j = 0; j < kPeGroup; ++j) {
                const int pe = g + j;
                if (pe >= npes) break;
#pragma unroll
                for (int u = 0; u < kReduceUnroll; ++u) {
                    if (pe == 0) {
                        acc[u] = x[j][u];
                    } else {
#pragma unroll
                        for (int k = 0; k < P::N; ++k)
                            acc[u].e[k] = nvshmemi_amd_fold_step<T, OP>(pe, acc[u].e[k], x[j][u].e[k]);
                    }
                }
            }
        }
        for (int pe = 0; pe < npes; ++pe) {
#pragma unroll
            for (int u = 0; u < kReduceUnroll; ++u) {
                const uint64_t v = v0 + (uint64_t)u * gsz;
                if (v < nvec) *reinterpret_cast<P *>(dst0 + (uint64_t)pe * pe_stride + 16 * v) = acc[u];
            }
        }
    }
    // elements behind the last full vector
    const uint64_t done = nvec * P::N;
    if (gid < nelems - done) {
        const uint64_t i = done + gid;
        const T *s = reinterpret_cast<const T *>(src0);
        T *d = reinterpret_cast<T *>(dst0);
        const uint64_t es = pe_stride / sizeof(T);
        T acc = s[i];
        for (int pe = 1; pe < npes; ++pe) acc = nvshmemi_amd_fold_step<T, OP>(pe, acc, s[(uint64_t)pe * es + i]);
        for (int pe = 0; pe < npes; ++pe) d[(uint64_t)pe * es + i] = acc;
    }
}

// Element-at-a-time variant for buffers that are not 16-byte aligned.
template <typename T, int OP>
__global__ __launch_bounds__(kThreads) void reduce_scalar_kernel(char *base, uint32_t shift, int npes,
                                                                 uint64_t dst_off, uint64_t src_off,
                                                                 uint64_t nelems) {
    const uint64_t gsz = (uint64_t)gridDim.x * kThreads;
    const uint64_t es = (1ull << shift) / sizeof(T);
    const T *s = reinterpret_cast<const T *>(base + src_off);
    T *d = reinterpret_cast<T *>(base + dst_off);
    for (uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x; i < nelems; i += gsz) {
        T acc = s[i];
        for (int pe = 1; pe < npes; ++pe) acc = nvshmemi_amd_fold_step<T, OP>(pe, acc, s[(uint64_t)pe * es + i]);
        for (int pe = 0; pe < npes; ++pe) d[(uint64_t)pe * es + i] = acc;
    }
}

template <typename T, int OP>
void launch_reduce(Runtime &rt, uint64_t dst_off, uint64_t src_off, uint64_t nelems,
                   hipStream_t stream) {
    const bool vector_ok = ((dst_off | src_off) & 15) == 0;
    const uint64_t per_thread = vector_ok ? (uint64_t)(16 / sizeof(T)) * kReduceUnroll : 1;
    uint64_t blocks = (nelems + per_thread * kThreads - 1) / (per_thread * kThreads);
    // enough resident work to cover HBM latency; more blocks than this only add launch cost
    const uint64_t cap = (uint64_t)rt.num_cus * 32;
    if (blocks > cap) blocks = cap;
    if (blocks == 0) blocks = 1;
    if (vector_ok)
        hipLaunchKernelGGL((reduce_vector_kernel<T, OP>), dim3((unsigned)blocks), dim3(kThreads), 0,
                           stream, rt.base, rt.heap_shift, rt.npes, dst_off, src_off, nelems);
    else
        hipLaunchKernelGGL((reduce_scalar_kernel<T, OP>), dim3((unsigned)blocks), dim3(kThreads), 0,
                           stream, rt.base, rt.heap_shift, rt.npes, dst_off, src_off, nelems);
}

typedef void (*reduce_launcher_t)(Runtime &, uint64_t, uint64_t, uint64_t, hipStream_t);

template <typename T>
reduce_launcher_t pick_arith(int op) {
    switch (op) {
        case NVSHMEMI_OP_min: return launch_reduce<T, NVSHMEMI_OP_min>;
        case NVSHMEMI_OP_max: return launch_reduce<T, NVSHMEMI_OP_max>;
        case NVSHMEMI_OP_sum: return launch_reduce<T, NVSHMEMI_OP_sum>;
        case NVSHMEMI_OP_prod: return launch_reduce<T, NVSHMEMI_OP_prod>;
        default: return nullptr;
    }
}
template <typename T>
reduce_launcher_t pick_integer(int op) {
    switch (op) {
        case NVSHMEMI_OP_and: return launch_reduce<T, NVSHMEMI_OP_and>;
        case NVSHMEMI_OP_or: return launch_reduce<T, NVSHMEMI_OP_or>;
        case NVSHMEMI_OP_xor: return launch_reduce<T, NVSHMEMI_OP_xor>;
        default: return pick_arith<T>(op);
    }
}

reduce_launcher_t pick_reduce(int dtype, int op) {
    switch (dtype) {
        case NVSHMEMI_DT_i8: return pick_integer<int8_t>(op);
        case NVSHMEMI_DT_i16: return pick_integer<int16_t>(op);
        case NVSHMEMI_DT_i32: return pick_integer<int32_t>(op);
        case NVSHMEMI_DT_i64: return pick_integer<int64_t>(op);
        case NVSHMEMI_DT_u8: return pick_integer<uint8_t>(op);
        case NVSHMEMI_DT_u16: return pick_integer<uint16_t>(op);
        case NVSHMEMI_DT_u32: return pick_integer<uint32_t>(op);
        case NVSHMEMI_DT_u64: return pick_integer<uint64_t>(op);
        case NVSHMEMI_DT_f16: return pick_arith<__half>(op);
        case NVSHMEMI_DT_bf16: return pick_arith<__hip_bfloat16>(op);
        case NVSHMEMI_DT_f32: return pick_arith<float>(op);
        case NVSHMEMI_DT_f64: return pick_arith<double>(op);
        default: return nullptr;
    }
}

const size_t kDtypeSize[NVSHMEMI_DT_COUNT] = {1, 2, 4, 8, 1, 2, 4, 8, 2, 2, 4, 8};

bool team_ok(Runtime &rt, const char *what, nvshmem_team_t team) {
    if (!rt.initialized) {
        set_error("%s called before nvshmem_init", what);
        return false;
    }
    if (team != NVSHMEM_TEAM_WORLD) {
        set_error("%s: team %d is not supported (only NVSHMEM_TEAM_WORLD)", what, (int)team);
        return false;
    }
    return true;
}

}  // namespace

int reduce_on_stream(int dtype, int op, nvshmem_team_t team, void *dest, const void *src,
                     size_t nreduce, hipStream_t stream) {
    Runtime &rt = Runtime::get();
    if (!team_ok(rt, "reduce", team)) return NVSHMEMX_ERROR_INVALID_VALUE;
    reduce_launcher_t fn = pick_reduce(dtype, op);
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
    fn(rt, doff, soff, nreduce, stream);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("reduce: kernel launch failed: %s", hipGetErrorString(e));
        return NVSHMEMX_ERROR_INTERNAL;
    }
    return 0;
}

static int segment_collective(int mode, const char *what, nvshmem_team_t team, void *dest,
                              const void *src, size_t seg_bytes, hipStream_t stream) {
    Runtime &rt = Runtime::get();
    if (!team_ok(rt, what, team)) return NVSHMEMX_ERROR_INVALID_VALUE;
    if (seg_bytes == 0) return 0;
    const uint64_t n = (uint64_t)rt.npes;
    if (seg_bytes > rt.heap_size / n) {
        set_error("%s: %zu bytes x %d PEs does not fit a PE's heap slice", what, seg_bytes, rt.npes);
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
    const uint64_t tiles = (seg_bytes / 16 + kTileVectors - 1) / kTileVectors + 1;
    const unsigned segs = mode == kModeFcollect ? (unsigned)n : (unsigned)(n * n);
    if (tiles > 0x7fffffffull) {
        set_error("%s: message too large", what);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    if (mode == kModeFcollect)
        hipLaunchKernelGGL((segment_copy_kernel<kModeFcollect>), dim3((unsigned)tiles, segs),
                           dim3(kThreads), 0, stream, rt.base, rt.heap_shift, rt.npes, doff, soff,
                           (uint64_t)seg_bytes);
    else
        hipLaunchKernelGGL((segment_copy_kernel<kModeAlltoall>), dim3((unsigned)tiles, segs),
                           dim3(kThreads), 0, stream, rt.base, rt.heap_shift, rt.npes, doff, soff,
                           (uint64_t)seg_bytes);
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
    }
NVSHMEMI_REPT_FOR_ALL_REDUCE_TYPES_AND_OPS(NVSHMEMI_DEFINE_TYPED_REDUCE_HOST)
#undef NVSHMEMI_DEFINE_TYPED_REDUCE_HOST

}  // extern "C"
