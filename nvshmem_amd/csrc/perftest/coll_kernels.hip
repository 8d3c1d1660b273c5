// In-kernel collectives through the public device API, one thread group per PE.
// Counterparts in the reference tree: perftest/device/coll/reduction_latency.cu:23-44,
// fcollect_latency.cu, alltoall_latency.cu, barrier_latency.cu (which time these calls from block 0
// of one kernel per PE and never check the result).
#include <hip/hip_runtime.h>

#include "nvshmem_perftest.h"
#include "nvshmemx.h"
#include "perftest_common.hpp"

namespace {

enum { kReduce = 0, kFcollect = 1, kAlltoall = 2 };

#define SCOPED_CALL(SCOPE, NAME, ...)                                               \
    do {                                                                            \
        if (SCOPE == NVSHMEM_PERFTEST_SCOPE_BLOCK) nvshmemx_##NAME##_block(__VA_ARGS__); \
        else if (SCOPE == NVSHMEM_PERFTEST_SCOPE_WARP) {                            \
            if (threadIdx.x < NVSHMEMI_WARP_SIZE) nvshmemx_##NAME##_warp(__VA_ARGS__); \
        } else {                                                                    \
            if (threadIdx.x == 0) nvshmem_##NAME(__VA_ARGS__);                      \
        }                                                                           \
    } while (0)

#define DEFINE_REDUCE_KERNEL(TNAME, TYPE, OP)                                                    \
    template <int SCOPE>                                                                         \
    __global__ void reduce_##TNAME##_##OP##_kernel(TYPE *dest, const TYPE *src, size_t n) {      \
        SCOPED_CALL(SCOPE, TNAME##_##OP##_reduce, NVSHMEM_TEAM_WORLD, dest, src, n);             \
    }
DEFINE_REDUCE_KERNEL(int32, int32_t, sum)
DEFINE_REDUCE_KERNEL(int64, int64_t, xor)
DEFINE_REDUCE_KERNEL(float, float, sum)
DEFINE_REDUCE_KERNEL(float, float, max)
DEFINE_REDUCE_KERNEL(bfloat16, nvshmem_bfloat16_t, sum)
DEFINE_REDUCE_KERNEL(bfloat16, nvshmem_bfloat16_t, max)
DEFINE_REDUCE_KERNEL(uint64, uint64_t, and)
DEFINE_REDUCE_KERNEL(double, double, prod)
DEFINE_REDUCE_KERNEL(int16, int16_t, min)

#define DEFINE_SCATTER_KERNEL(TNAME, TYPE, OP)                                                   \
    template <int SCOPE>                                                                         \
    __global__ void reducescatter_##TNAME##_##OP##_kernel(TYPE *dest, const TYPE *src, size_t n) { \
        SCOPED_CALL(SCOPE, TNAME##_##OP##_reducescatter, NVSHMEM_TEAM_WORLD, dest, src, n);      \
    }
DEFINE_SCATTER_KERNEL(int32, int32_t, sum)
DEFINE_SCATTER_KERNEL(float, float, sum)
DEFINE_SCATTER_KERNEL(float, float, max)
DEFINE_SCATTER_KERNEL(bfloat16, nvshmem_bfloat16_t, sum)
DEFINE_SCATTER_KERNEL(uint64, uint64_t, xor)

template <int SCOPE>
__global__ void broadcast_kernel(char *dest, const char *src, size_t bytes, int root) {
    SCOPED_CALL(SCOPE, broadcastmem, NVSHMEM_TEAM_WORLD, dest, src, bytes, root);
}
template <int SCOPE>
__global__ void fcollect_kernel(char *dest, const char *src, size_t bytes) {
    SCOPED_CALL(SCOPE, fcollectmem, NVSHMEM_TEAM_WORLD, dest, src, bytes);
}
template <int SCOPE>
__global__ void alltoall_kernel(char *dest, const char *src, size_t bytes) {
    SCOPED_CALL(SCOPE, alltoallmem, NVSHMEM_TEAM_WORLD, dest, src, bytes);
}

template <int SCOPE>
__global__ void barrier_kernel(uint64_t *counter, uint64_t *errors, int rounds) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    uint64_t *my_counter = (uint64_t *)nvshmem_ptr(counter, me);
    uint64_t bad = 0;
    for (int r = 1; r <= rounds; ++r) {
        if (threadIdx.x == 0) *my_counter = (uint64_t)r;
        SCOPED_CALL(SCOPE, barrier_all);
        if (threadIdx.x == 0)
            for (int q = 0; q < np; ++q) bad += nvshmem_uint64_g(counter, q) < (uint64_t)r;
        // nobody may start round r+1 (and overwrite its counter) while others still check round r
        SCOPED_CALL(SCOPE, barrier_all);
    }
    if (threadIdx.x == 0) *(uint64_t *)nvshmem_ptr(errors, me) += bad;
}

// Collectives and queries on a team handle; PEs that are not members of `team` return at once.
enum { kTeamReduce = 0, kTeamReducescatter = 1, kTeamFcollect = 2, kTeamAlltoall = 3, kTeamBroadcast = 4,
       kTeamBarrier = 5, kTeamSync = 6 };

// `iters` > 1 repeats the call inside the kernel, which is how the reference's device perftests
// time a collective (perftest/device/coll/*_latency.cu): the launch is paid once.
template <int SCOPE>
__global__ void team_coll_kernel(int what, nvshmem_team_t team, void *dest, const void *src, size_t n,
                                 int root, int iters) {
    if (nvshmem_team_my_pe(team) < 0) return;
    for (int it = 0; it < iters; ++it) switch (what) {
        case kTeamReduce:
            SCOPED_CALL(SCOPE, float_sum_reduce, team, (float *)dest, (const float *)src, n);
            break;
        case kTeamReducescatter:
            SCOPED_CALL(SCOPE, float_sum_reducescatter, team, (float *)dest, (const float *)src, n);
            break;
        case kTeamFcollect: SCOPED_CALL(SCOPE, fcollectmem, team, dest, src, n); break;
        case kTeamAlltoall: SCOPED_CALL(SCOPE, alltoallmem, team, dest, src, n); break;
        case kTeamBarrier: SCOPED_CALL(SCOPE, barrier, team); break;
        case kTeamSync: SCOPED_CALL(SCOPE, team_sync, team); break;
        default: SCOPED_CALL(SCOPE, broadcastmem, team, dest, src, n, root); break;
    }
}

// (value, location) maximum among the members of `team`, `iters` times; thread 0 of every PE also
// stores what the device-side identification calls report into info[0..3] (major, minor of the
// specification, then vendor major * 10000 + minor * 100 + patch, then the length of the name).
__global__ void maxloc_kernel(nvshmem_team_t team, double2 *dest, const double2 *src, size_t n, int iters,
                              int *info) {
    if (threadIdx.x == 0 && info) {
        int *mine = (int *)nvshmem_ptr(info, nvshmem_my_pe());
        int major = 0, minor = 0, patch = 0;
        nvshmem_info_get_version(&mine[0], &mine[1]);
        nvshmemx_vendor_get_version_info(&major, &minor, &patch);
        mine[2] = major * 10000 + minor * 100 + patch;
        char name[NVSHMEM_MAX_NAME_LEN];
        nvshmem_info_get_name(name);
        int len = 0;
        while (len < NVSHMEM_MAX_NAME_LEN && name[len]) ++len;
        mine[3] = len;
    }
    if (nvshmem_team_my_pe(team) < 0) return;
    for (int it = 0; it < iters; ++it) nvshmemx_double2_maxloc_reduce_block(team, dest, src, n);
}

// out (symmetric, 4 + NVSHMEMI_AMD_MAX_PES ints per PE): my_pe(a), n_pes(a), my_pe(b), n_pes(b),
// then translate_pe(a, i, b) for i = 0 .. NVSHMEMI_AMD_MAX_PES-1
__global__ void team_query_kernel(int *out, nvshmem_team_t a, nvshmem_team_t b) {
    if (threadIdx.x != 0) return;
    int *mine = (int *)nvshmem_ptr(out, nvshmem_my_pe());
    mine[0] = nvshmem_team_my_pe(a);
    mine[1] = nvshmem_team_n_pes(a);
    mine[2] = nvshmem_team_my_pe(b);
    mine[3] = nvshmem_team_n_pes(b);
    for (int i = 0; i < NVSHMEMI_AMD_MAX_PES; ++i) mine[4 + i] = nvshmem_team_translate_pe(a, i, b);
}

// Team barrier check: like barrier_kernel, but only among the members of `team`, whose counters
// are read through the team's PE translation.
template <int SCOPE>
__global__ void team_barrier_kernel(uint64_t *counter, uint64_t *errors, int rounds, nvshmem_team_t team) {
    const int idx = nvshmem_team_my_pe(team), np = nvshmem_team_n_pes(team);
    if (idx < 0) return;
    const int me = nvshmem_my_pe();
    uint64_t *my_counter = (uint64_t *)nvshmem_ptr(counter, me);
    uint64_t bad = 0;
    for (int r = 1; r <= rounds; ++r) {
        if (threadIdx.x == 0) *my_counter = (uint64_t)r;
        SCOPED_CALL(SCOPE, barrier, team);
        if (threadIdx.x == 0)
            for (int q = 0; q < np; ++q)
                bad += nvshmem_uint64_g(counter, nvshmem_team_translate_pe(team, q, NVSHMEM_TEAM_WORLD)) < (uint64_t)r;
        SCOPED_CALL(SCOPE, team_sync, team);
    }
    if (threadIdx.x == 0) *(uint64_t *)nvshmem_ptr(errors, me) += bad;
}

// nvshmemx_barrier_warpgroup: warpgroup `group` (threads [256 group, 256 group + 256) of the block) of
// every member runs the rounds of team_barrier_kernel; the other threads of the block leave at once.
__global__ void warpgroup_barrier_kernel(uint64_t *counter, uint64_t *errors, int rounds, nvshmem_team_t team,
                                         int group) {
    const int idx = nvshmem_team_my_pe(team), np = nvshmem_team_n_pes(team);
    if (idx < 0 || (int)(threadIdx.x / NVSHMEMI_AMD_WARPGROUP_SIZE) != group) return;
    const unsigned local = threadIdx.x % NVSHMEMI_AMD_WARPGROUP_SIZE;
    const unsigned rest = blockDim.x - group * NVSHMEMI_AMD_WARPGROUP_SIZE;
    const unsigned members = rest < NVSHMEMI_AMD_WARPGROUP_SIZE ? rest : NVSHMEMI_AMD_WARPGROUP_SIZE;
    const bool leader = local == 0;
    const int me = nvshmem_my_pe();
    uint64_t *my_counter = (uint64_t *)nvshmem_ptr(counter, me);
    uint64_t bad = 0;
    for (int r = 1; r <= rounds; ++r) {
        // the LAST thread of the warpgroup writes and the first one checks: the barrier has to order the
        // wavefronts of the group as well as the PEs
        if (local == members - 1) *my_counter = (uint64_t)r;
        nvshmemx_barrier_warpgroup(team);
        if (leader)
            for (int q = 0; q < np; ++q)
                bad += nvshmem_uint64_g(counter, nvshmem_team_translate_pe(team, q, NVSHMEM_TEAM_WORLD)) < (uint64_t)r;
        nvshmemx_barrier_warpgroup(team);
    }
    if (leader) *(uint64_t *)nvshmem_ptr(errors, me) += bad;
}

// Many collectives back to back without any barrier in between (sync_between = 0) or with one
// after every check (1): round r fills src[i] = gen(me, r, i), then runs an int32 sum reduce of n
// elements, a broadcast of the same n elements from member r % npes, an fcollect of fc_bytes per
// PE, and - when n >= npes - an alltoall and a reducescatter of n / npes words per member, all into
// dst, and folds a position-weighted checksum of dst into check[0] after each.
__device__ inline int32_t ll_gen(int me, int r, int i) {
    return (int32_t)(((uint32_t)me * 1000003u + (uint32_t)r * 7919u + (uint32_t)i * 31u) & 0x7fffffffu);
}
__device__ inline uint64_t ll_checksum(uint64_t h, const int32_t *words, size_t n) {
    uint64_t s = 0;
    for (size_t i = 0; i < n; ++i) s += (uint64_t)(uint32_t)words[i] * (2 * (uint64_t)i + 1);
    return h * 1000003ull + s;
}
template <int SCOPE>
__global__ void coll_sequence_kernel(int32_t *src, int32_t *dst, uint64_t *check, int n, int fc_bytes,
                                     int rounds, int sync_between) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    int32_t *my_src = (int32_t *)nvshmem_ptr(src, me);
    const int32_t *my_dst = (const int32_t *)nvshmem_ptr(dst, me);
    uint64_t h = 0;
    for (int r = 0; r < rounds; ++r) {
        for (int i = threadIdx.x; i < n; i += blockDim.x) my_src[i] = ll_gen(me, r, i);
        __syncthreads();
        SCOPED_CALL(SCOPE, int32_sum_reduce, NVSHMEM_TEAM_WORLD, dst, src, (size_t)n);
        __syncthreads();
        if (threadIdx.x == 0) h = ll_checksum(h, my_dst, (size_t)n);
        __syncthreads();
        if (sync_between) SCOPED_CALL(SCOPE, barrier_all);
        SCOPED_CALL(SCOPE, broadcastmem, NVSHMEM_TEAM_WORLD, dst, src, (size_t)n * 4, r % np);
        __syncthreads();
        if (threadIdx.x == 0) h = ll_checksum(h, my_dst, (size_t)n);
        __syncthreads();
        if (sync_between) SCOPED_CALL(SCOPE, barrier_all);
        SCOPED_CALL(SCOPE, fcollectmem, NVSHMEM_TEAM_WORLD, dst, src, (size_t)fc_bytes);
        __syncthreads();
        if (threadIdx.x == 0) h = ll_checksum(h, my_dst, (size_t)fc_bytes * np / 4);
        __syncthreads();
        if (sync_between) SCOPED_CALL(SCOPE, barrier_all);
        // alltoall of a2a_words per destination and reducescatter of the same count, both out of
        // the first np * a2a_words words of src
        const size_t a2a_words = (size_t)n / (size_t)np;
        if (a2a_words) {
            SCOPED_CALL(SCOPE, alltoallmem, NVSHMEM_TEAM_WORLD, dst, src, a2a_words * 4);
            __syncthreads();
            if (threadIdx.x == 0) h = ll_checksum(h, my_dst, a2a_words * np);
            __syncthreads();
            if (sync_between) SCOPED_CALL(SCOPE, barrier_all);
            SCOPED_CALL(SCOPE, int32_sum_reducescatter, NVSHMEM_TEAM_WORLD, dst, src, a2a_words);
            __syncthreads();
            if (threadIdx.x == 0) h = ll_checksum(h, my_dst, a2a_words);
            __syncthreads();
            if (sync_between) SCOPED_CALL(SCOPE, barrier_all);
        }
    }
    if (threadIdx.x == 0) *(uint64_t *)nvshmem_ptr(check, me) = h;
}

template <typename... Args>
int launch_scoped(int scope, void (*kb)(Args...), void (*kw)(Args...), void (*kt)(Args...),
                  int threads, void *stream, Args... a) {
    void *args[] = {(void *)&a...};
    const void *fn = scope == NVSHMEM_PERFTEST_SCOPE_BLOCK  ? (const void *)kb
                     : scope == NVSHMEM_PERFTEST_SCOPE_WARP ? (const void *)kw
                                                            : (const void *)kt;
    return nvshmemx_collective_launch(fn, dim3(1), dim3(threads), args, 0, (hipStream_t)stream);
}

#define LAUNCH_REDUCE(TNAME, TYPE, OP)                                                           \
    return launch_scoped<TYPE *, const TYPE *, size_t>(                                          \
        scope, reduce_##TNAME##_##OP##_kernel<NVSHMEM_PERFTEST_SCOPE_BLOCK>,                     \
        reduce_##TNAME##_##OP##_kernel<NVSHMEM_PERFTEST_SCOPE_WARP>,                             \
        reduce_##TNAME##_##OP##_kernel<NVSHMEM_PERFTEST_SCOPE_THREAD>, threads, stream,          \
        (TYPE *)dest, (const TYPE *)src, nreduce)

#define LAUNCH_SCATTER(TNAME, TYPE, OP)                                                          \
    return launch_scoped<TYPE *, const TYPE *, size_t>(                                          \
        scope, reducescatter_##TNAME##_##OP##_kernel<NVSHMEM_PERFTEST_SCOPE_BLOCK>,              \
        reducescatter_##TNAME##_##OP##_kernel<NVSHMEM_PERFTEST_SCOPE_WARP>,                      \
        reducescatter_##TNAME##_##OP##_kernel<NVSHMEM_PERFTEST_SCOPE_THREAD>, threads, stream,   \
        (TYPE *)dest, (const TYPE *)src, nreduce)

}  // namespace

extern "C" {

int nvshmem_perftest_unit_packets_compiled(void) {
#ifdef NVSHMEMI_AMD_UNIT_PACKETS
    return 1;
#else
    return 0;
#endif
}

int nvshmem_perftest_device_reducescatter(int dtype, int op, void *dest, const void *src,
                                          size_t nreduce, int scope, int threads, void *stream) {
    static const size_t esize[NVSHMEMI_DT_COUNT] = {1, 2, 4, 8, 1, 2, 4, 8, 2, 2, 4, 8};
    if (!perftest::ready() || dtype < 0 || dtype >= NVSHMEMI_DT_COUNT || scope < 0 || scope > 2 ||
        !perftest::check_launch(1, threads) || !perftest::check_range(dest, nreduce * esize[dtype]) ||
        !perftest::check_range(src, nreduce * esize[dtype] * (size_t)nvshmem_n_pes()))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    const int key = dtype * 16 + op;
    switch (key) {
        case NVSHMEMI_DT_i32 * 16 + NVSHMEMI_OP_sum: LAUNCH_SCATTER(int32, int32_t, sum);
        case NVSHMEMI_DT_f32 * 16 + NVSHMEMI_OP_sum: LAUNCH_SCATTER(float, float, sum);
        case NVSHMEMI_DT_f32 * 16 + NVSHMEMI_OP_max: LAUNCH_SCATTER(float, float, max);
        case NVSHMEMI_DT_bf16 * 16 + NVSHMEMI_OP_sum: LAUNCH_SCATTER(bfloat16, nvshmem_bfloat16_t, sum);
        case NVSHMEMI_DT_u64 * 16 + NVSHMEMI_OP_xor: LAUNCH_SCATTER(uint64, uint64_t, xor);
        default: return NVSHMEMX_ERROR_NOT_SUPPORTED;
    }
}

int nvshmem_perftest_device_broadcast(void *dest, const void *src, size_t bytes, int root,
                                      int scope, int threads, void *stream) {
    if (!perftest::ready() || scope < 0 || scope > 2 || root < 0 || root >= nvshmem_n_pes() ||
        !perftest::check_launch(1, threads) || !perftest::check_range(dest, bytes) ||
        !perftest::check_range(src, bytes))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    return launch_scoped<char *, const char *, size_t, int>(
        scope, broadcast_kernel<NVSHMEM_PERFTEST_SCOPE_BLOCK>, broadcast_kernel<NVSHMEM_PERFTEST_SCOPE_WARP>,
        broadcast_kernel<NVSHMEM_PERFTEST_SCOPE_THREAD>, threads, stream, (char *)dest,
        (const char *)src, bytes, root);
}

int nvshmem_perftest_device_reduce(int dtype, int op, void *dest, const void *src, size_t nreduce,
                                   int scope, int threads, void *stream) {
    static const size_t esize[NVSHMEMI_DT_COUNT] = {1, 2, 4, 8, 1, 2, 4, 8, 2, 2, 4, 8};
    if (!perftest::ready() || dtype < 0 || dtype >= NVSHMEMI_DT_COUNT || scope < 0 || scope > 2 ||
        !perftest::check_launch(1, threads) || !perftest::check_range(dest, nreduce * esize[dtype]) ||
        !perftest::check_range(src, nreduce * esize[dtype]))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    const int key = dtype * 16 + op;
    switch (key) {
        case NVSHMEMI_DT_i32 * 16 + NVSHMEMI_OP_sum: LAUNCH_REDUCE(int32, int32_t, sum);
        case NVSHMEMI_DT_i64 * 16 + NVSHMEMI_OP_xor: LAUNCH_REDUCE(int64, int64_t, xor);
        case NVSHMEMI_DT_f32 * 16 + NVSHMEMI_OP_sum: LAUNCH_REDUCE(float, float, sum);
        case NVSHMEMI_DT_f32 * 16 + NVSHMEMI_OP_max: LAUNCH_REDUCE(float, float, max);
        case NVSHMEMI_DT_bf16 * 16 + NVSHMEMI_OP_sum: LAUNCH_REDUCE(bfloat16, nvshmem_bfloat16_t, sum);
        case NVSHMEMI_DT_bf16 * 16 + NVSHMEMI_OP_max: LAUNCH_REDUCE(bfloat16, nvshmem_bfloat16_t, max);
        case NVSHMEMI_DT_u64 * 16 + NVSHMEMI_OP_and: LAUNCH_REDUCE(uint64, uint64_t, and);
        case NVSHMEMI_DT_f64 * 16 + NVSHMEMI_OP_prod: LAUNCH_REDUCE(double, double, prod);
        case NVSHMEMI_DT_i16 * 16 + NVSHMEMI_OP_min: LAUNCH_REDUCE(int16, int16_t, min);
        default: return NVSHMEMX_ERROR_NOT_SUPPORTED;
    }
}

int nvshmem_perftest_device_fcollect(void *dest, const void *src, size_t bytes, int scope,
                                     int threads, void *stream) {
    if (!perftest::ready() || scope < 0 || scope > 2 || !perftest::check_launch(1, threads) ||
        !perftest::check_range(dest, bytes * (size_t)nvshmem_n_pes()) ||
        !perftest::check_range(src, bytes))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    return launch_scoped<char *, const char *, size_t>(
        scope, fcollect_kernel<NVSHMEM_PERFTEST_SCOPE_BLOCK>, fcollect_kernel<NVSHMEM_PERFTEST_SCOPE_WARP>,
        fcollect_kernel<NVSHMEM_PERFTEST_SCOPE_THREAD>, threads, stream, (char *)dest,
        (const char *)src, bytes);
}

int nvshmem_perftest_device_alltoall(void *dest, const void *src, size_t bytes, int scope,
                                     int threads, void *stream) {
    const size_t total = bytes * (size_t)nvshmem_n_pes();
    if (!perftest::ready() || scope < 0 || scope > 2 || !perftest::check_launch(1, threads) ||
        !perftest::check_range(dest, total) || !perftest::check_range(src, total))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    return launch_scoped<char *, const char *, size_t>(
        scope, alltoall_kernel<NVSHMEM_PERFTEST_SCOPE_BLOCK>, alltoall_kernel<NVSHMEM_PERFTEST_SCOPE_WARP>,
        alltoall_kernel<NVSHMEM_PERFTEST_SCOPE_THREAD>, threads, stream, (char *)dest,
        (const char *)src, bytes);
}

int nvshmem_perftest_device_barrier(uint64_t *counter, uint64_t *errors, int rounds, int scope,
                                    int threads, void *stream) {
    if (!perftest::ready() || scope < 0 || scope > 2 || !perftest::check_launch(1, threads) ||
        !perftest::check_range(counter, sizeof(uint64_t)) ||
        !perftest::check_range(errors, sizeof(uint64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    return launch_scoped<uint64_t *, uint64_t *, int>(
        scope, barrier_kernel<NVSHMEM_PERFTEST_SCOPE_BLOCK>, barrier_kernel<NVSHMEM_PERFTEST_SCOPE_WARP>,
        barrier_kernel<NVSHMEM_PERFTEST_SCOPE_THREAD>, threads, stream, counter, errors, rounds);
}

int nvshmem_perftest_device_team_coll_loop(int what, int team, void *dest, const void *src,
                                           size_t n, int root, int iters, int scope, int threads,
                                           void *stream) {
    if (!perftest::ready() || scope < 0 || scope > 2 || what < kTeamReduce || what > kTeamSync ||
        iters < 1 || !perftest::check_launch(1, threads) || !perftest::check_range(dest, 1) ||
        !perftest::check_range(src, 1))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    return launch_scoped<int, nvshmem_team_t, void *, const void *, size_t, int, int>(
        scope, team_coll_kernel<NVSHMEM_PERFTEST_SCOPE_BLOCK>, team_coll_kernel<NVSHMEM_PERFTEST_SCOPE_WARP>,
        team_coll_kernel<NVSHMEM_PERFTEST_SCOPE_THREAD>, threads, stream, what, (nvshmem_team_t)team,
        dest, src, n, root, iters);
}

int nvshmem_perftest_device_team_coll(int what, int team, void *dest, const void *src, size_t n,
                                      int root, int scope, int threads, void *stream) {
    if (what >= kTeamBarrier) return NVSHMEMX_ERROR_INVALID_VALUE;
    return nvshmem_perftest_device_team_coll_loop(what, team, dest, src, n, root, 1, scope, threads,
                                                  stream);
}

int nvshmem_perftest_device_maxloc(int team, void *dest, const void *src, size_t nreduce, int iters,
                                   int threads, int *info, void *stream) {
    if (!perftest::ready() || iters < 1 || !perftest::check_launch(1, threads) ||
        !perftest::check_range(dest, nreduce * sizeof(double2)) ||
        !perftest::check_range(src, nreduce * sizeof(double2)) ||
        (info && !perftest::check_range(info, 4 * sizeof(int))))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    nvshmem_team_t t = team;
    double2 *d = (double2 *)dest;
    const double2 *s = (const double2 *)src;
    void *args[] = {(void *)&t, (void *)&d, (void *)&s, (void *)&nreduce, (void *)&iters, (void *)&info};
    return nvshmemx_collective_launch((const void *)maxloc_kernel, dim3(1), dim3(threads), args, 0,
                                      (hipStream_t)stream);
}

int nvshmem_perftest_team_query(int *out, int team_a, int team_b, void *stream) {
    if (!perftest::ready() ||
        !perftest::check_range(out, sizeof(int) * (4 + NVSHMEMI_AMD_MAX_PES)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    nvshmem_team_t a = team_a, b = team_b;
    void *args[] = {(void *)&out, (void *)&a, (void *)&b};
    return nvshmemx_collective_launch((const void *)team_query_kernel, dim3(1), dim3(64), args, 0,
                                      (hipStream_t)stream);
}

int nvshmem_perftest_device_team_barrier(uint64_t *counter, uint64_t *errors, int rounds, int team,
                                         int scope, int threads, void *stream) {
    if (!perftest::ready() || scope < 0 || scope > 2 || !perftest::check_launch(1, threads) ||
        !perftest::check_range(counter, sizeof(uint64_t)) ||
        !perftest::check_range(errors, sizeof(uint64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    return launch_scoped<uint64_t *, uint64_t *, int, nvshmem_team_t>(
        scope, team_barrier_kernel<NVSHMEM_PERFTEST_SCOPE_BLOCK>,
        team_barrier_kernel<NVSHMEM_PERFTEST_SCOPE_WARP>, team_barrier_kernel<NVSHMEM_PERFTEST_SCOPE_THREAD>,
        threads, stream, counter, errors, rounds, (nvshmem_team_t)team);
}

int nvshmem_perftest_device_warpgroup_barrier(uint64_t *counter, uint64_t *errors, int rounds, int team,
                                              int group, int threads, void *stream) {
    if (!perftest::ready() || !perftest::check_launch(1, threads) || group < 0 ||
        group * NVSHMEMI_AMD_WARPGROUP_SIZE >= threads ||
        !perftest::check_range(counter, sizeof(uint64_t)) || !perftest::check_range(errors, sizeof(uint64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    nvshmem_team_t t = team;
    void *args[] = {(void *)&counter, (void *)&errors, (void *)&rounds, (void *)&t, (void *)&group};
    return nvshmemx_collective_launch((const void *)warpgroup_barrier_kernel, dim3(1), dim3(threads), args, 0,
                                      (hipStream_t)stream);
}

int nvshmem_perftest_coll_sequence(int32_t *src, int32_t *dst, uint64_t *check, int n, int fc_bytes,
                                   int rounds, int sync_between, int scope, int threads, void *stream) {
    const size_t np = (size_t)nvshmem_n_pes();
    if (!perftest::ready() || scope < 0 || scope > 2 || n < 1 || fc_bytes < 4 || fc_bytes % 4 ||
        rounds < 1 || !perftest::check_launch(1, threads) ||
        !perftest::check_range(src, (size_t)n * 4 > (size_t)fc_bytes ? (size_t)n * 4 : (size_t)fc_bytes) ||
        !perftest::check_range(dst, (size_t)n * 4 > fc_bytes * np ? (size_t)n * 4 : fc_bytes * np) ||
        !perftest::check_range(check, sizeof(uint64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if ((size_t)fc_bytes > (size_t)n * 4) return NVSHMEMX_ERROR_INVALID_VALUE;  // fcollect sends src[0, fc_bytes)
    return launch_scoped<int32_t *, int32_t *, uint64_t *, int, int, int, int>(
        scope, coll_sequence_kernel<NVSHMEM_PERFTEST_SCOPE_BLOCK>,
        coll_sequence_kernel<NVSHMEM_PERFTEST_SCOPE_WARP>, coll_sequence_kernel<NVSHMEM_PERFTEST_SCOPE_THREAD>,
        threads, stream, src, dst, check, n, fc_bytes, rounds, sync_between);
}

}  // extern "C"
