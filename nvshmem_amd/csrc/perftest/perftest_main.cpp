// Command-line performance driver over the public C ABI, with the conventions of the reference's
// perftest programs (perftest/common/utils.cu:661-689 table layout; warm-up then timed iterations
// between events; sizes doubling from --min to --max; bandwidth = payload bytes / time as in
// perftest/device/pt-to-pt/shmem_put_bw.cu:118-128, latency in microseconds as in
// perftest/device/coll/*_latency.cu).
//
//   nvshmem_perftest <test> [--npes N] [--min BYTES] [--max BYTES] [--iters K] [--warmup W]
//                           [--blocks B] [--threads T] [--scope thread|warp|block] [--elem 1|2|4|8] [--graph]
//
// tests: put_bw get_bw                      device put/get, every PE to its right neighbour
//        p_bw g_bw st_bw atomic_bw          one element per thread and call (--elem 1|2|4|8 bytes):
//                                           nvshmem_<T>_p / _g, a plain store through nvshmem_ptr,
//                                           nvshmem_<T>_atomic_add
//        reduce reducescatter fcollect alltoall broadcast
//                                           host-launched collectives on a stream (fp32 sum for the
//                                           reductions); size = bytes each PE contributes; --graph
//                                           captures the timed calls in one HIP graph and replays it
//        coll_latency                       the same five calls made inside a kernel, the call
//                                           repeated --iters times in one launch
//        barrier_latency sync_latency       nvshmem_barrier_all / nvshmem_sync_all inside a kernel
//        barrier_on_stream sync_on_stream   nvshmemx_barrier_all_on_stream / nvshmemx_sync_all_on_stream and
//                                           their team forms (perftest/host/coll/barrier_on_stream.cpp)
//        malloc                             nvshmem_malloc / nvshmem_free of doubling sizes
//                                           (perftest/host/init/malloc.cpp)
//        host_put_bw host_get_bw            nvshmemx_putmem_on_stream / getmem_on_stream from PE 0 to
//                                           PE 1 (perftest/host/pt-to-pt/bw.cpp)
//        pt2pt_latency                      put / get (+ put_signal ping-pong) latency per size and
//                                           p, g, fetching atomic, signal / p / atomic ping-pong
//                                           latency between PE 0 and PE 1, inside one kernel
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <string>
#include <vector>

#include "nvshmem.h"
#include "nvshmem_perftest.h"

namespace {

struct Options {
    std::string test;
    int npes = 8;
    size_t min_bytes = 8, max_bytes = (size_t)64 << 20;
    int iters = 20, warmup = 5;
    int blocks = 0, threads = 0;  // 0: a shape that fills the GPU
    int scope = NVSHMEM_PERFTEST_SCOPE_BLOCK;
    int elem = 8;  // element size of the element-wise tests
    bool graph = false;  // host collectives: capture the timed calls in one HIP graph
};

[[noreturn]] void usage(const char *why) {
    fprintf(stderr, "nvshmem_perftest: %s\nusage: nvshmem_perftest <put_bw|get_bw|p_bw|g_bw|st_bw|atomic_bw|reduce|reducescatter|fcollect|"
                    "alltoall|broadcast|coll_latency|barrier_latency|sync_latency|barrier_on_stream|sync_on_stream|pt2pt_latency|host_put_bw|host_get_bw|malloc> [--npes N] [--min B] [--max B] [--iters K] "
                    "[--warmup W] [--blocks B] [--threads T] [--scope thread|warp|block] [--elem 1|2|4|8] [--graph]\n", why);
    exit(2);
}

size_t parse_size(const char *s) {
    char *end = nullptr;
    double v = strtod(s, &end);
    if (end == s || v < 0) usage("bad size");
    switch (*end) {
        case 'k': case 'K': v *= 1024.0; break;
        case 'm': case 'M': v *= 1024.0 * 1024.0; break;
        case 'g': case 'G': v *= 1024.0 * 1024.0 * 1024.0; break;
        default: break;
    }
    return (size_t)v;
}

Options parse(int argc, char **argv) {
    if (argc < 2) usage("no test named");
    Options o;
    o.test = argv[1];
    for (int i = 2; i < argc; ++i) {
        const std::string a = argv[i];
        auto next = [&]() -> const char * {
            if (i + 1 >= argc) usage(("missing value after " + a).c_str());
            return argv[++i];
        };
        if (a == "--npes") o.npes = atoi(next());
        else if (a == "--min") o.min_bytes = parse_size(next());
        else if (a == "--max") o.max_bytes = parse_size(next());
        else if (a == "--iters") o.iters = atoi(next());
        else if (a == "--warmup") o.warmup = atoi(next());
        else if (a == "--blocks") o.blocks = atoi(next());
        else if (a == "--threads") o.threads = atoi(next());
        else if (a == "--elem") o.elem = atoi(next());
        else if (a == "--graph") o.graph = true;
        else if (a == "--scope") {
            const std::string s = next();
            if (s == "thread") o.scope = NVSHMEM_PERFTEST_SCOPE_THREAD;
            else if (s == "warp") o.scope = NVSHMEM_PERFTEST_SCOPE_WARP;
            else if (s == "block") o.scope = NVSHMEM_PERFTEST_SCOPE_BLOCK;
            else usage("bad scope");
        } else usage(("unknown option " + a).c_str());
    }
    if (o.iters < 1 || o.warmup < 0 || o.min_bytes < 1 || o.max_bytes < o.min_bytes) usage("bad range");
    if (o.elem != 1 && o.elem != 2 && o.elem != 4 && o.elem != 8) usage("bad element size");
    if (o.test == "atomic_bw" && o.elem < 4) usage("atomics are 4 or 8 bytes wide");
    return o;
}

const char *scope_name(int scope) {
    return scope == NVSHMEM_PERFTEST_SCOPE_THREAD ? "thread" : scope == NVSHMEM_PERFTEST_SCOPE_WARP ? "warp" : "block";
}

#define CHECK_HIP(x)                                                                         \
    do {                                                                                     \
        hipError_t e_ = (x);                                                                 \
        if (e_ != hipSuccess) {                                                              \
            fprintf(stderr, "%s failed: %s (%s:%d)\n", #x, hipGetErrorString(e_), __FILE__, __LINE__); \
            exit(1);                                                                         \
        }                                                                                    \
    } while (0)

// average milliseconds of one call of fn: `warmup` untimed calls, then `iters` between two events
template <typename Fn>
double time_ms(Fn fn, int iters, int warmup) {
    for (int i = 0; i < warmup; ++i)
        if (fn() != 0) {
            fprintf(stderr, "nvshmem_perftest: call failed: %s\n", nvshmemx_amd_last_error());
            exit(1);
        }
    CHECK_HIP(hipDeviceSynchronize());
    hipEvent_t a, b;
    CHECK_HIP(hipEventCreate(&a));
    CHECK_HIP(hipEventCreate(&b));
    CHECK_HIP(hipEventRecord(a, nullptr));
    for (int i = 0; i < iters; ++i) (void)fn();
    CHECK_HIP(hipEventRecord(b, nullptr));
    CHECK_HIP(hipEventSynchronize(b));
    float ms = 0;
    CHECK_HIP(hipEventElapsedTime(&ms, a, b));
    CHECK_HIP(hipEventDestroy(a));
    CHECK_HIP(hipEventDestroy(b));
    return (double)ms / iters;
}

// The same measurement with the `iters` calls captured once into a HIP graph on `stream` and replayed
// (the graph variant of the reference's host collective tests, perftest/host/coll/coll_test.h:128-186):
// average milliseconds per captured call over `replays` replays after one warm-up replay.
template <typename Fn>
double time_graph_ms(Fn fn, int iters, hipStream_t stream, int replays = 5) {
    hipGraph_t graph;
    hipGraphExec_t exec;
    CHECK_HIP(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal));
    for (int i = 0; i < iters; ++i)
        if (fn() != 0) {
            fprintf(stderr, "nvshmem_perftest: call failed under capture: %s\n", nvshmemx_amd_last_error());
            exit(1);
        }
    CHECK_HIP(hipStreamEndCapture(stream, &graph));
    CHECK_HIP(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    CHECK_HIP(hipGraphLaunch(exec, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    hipEvent_t a, b;
    CHECK_HIP(hipEventCreate(&a));
    CHECK_HIP(hipEventCreate(&b));
    CHECK_HIP(hipEventRecord(a, stream));
    for (int r = 0; r < replays; ++r) CHECK_HIP(hipGraphLaunch(exec, stream));
    CHECK_HIP(hipEventRecord(b, stream));
    CHECK_HIP(hipEventSynchronize(b));
    float ms = 0;
    CHECK_HIP(hipEventElapsedTime(&ms, a, b));
    CHECK_HIP(hipEventDestroy(a));
    CHECK_HIP(hipEventDestroy(b));
    CHECK_HIP(hipGraphExecDestroy(exec));
    CHECK_HIP(hipGraphDestroy(graph));
    return (double)ms / replays / iters;
}

void print_table(const char *job, const char *scope, const char *what, const char *units,
                 const std::vector<size_t> &sizes, const std::vector<double> &values) {
    char head[64];
    snprintf(head, sizeof head, "%s (%s)", what, units);
    printf("#%10s\n%-10s  %-8s  %-16s\n", job, "size(B)", "scope", head);
    for (size_t i = 0; i < sizes.size(); ++i) printf("%-10zu  %-8s  %-16.6f\n", sizes[i], scope, values[i]);
}

std::vector<size_t> sweep(const Options &o, size_t multiple) {
    std::vector<size_t> out;
    for (size_t s = o.min_bytes; s <= o.max_bytes; s *= 2) {
        const size_t r = (s + multiple - 1) / multiple * multiple;
        if (out.empty() || out.back() != r) out.push_back(r);
    }
    return out;
}

int run_rma(const Options &o, bool is_get) {
    void *src = nvshmem_malloc(o.max_bytes), *dst = nvshmem_malloc(o.max_bytes);
    if (!src || !dst) return 1;
    std::vector<size_t> sizes = sweep(o, 1);
    std::vector<double> gbs;
    for (size_t bytes : sizes) {
        // default: a block of one wavefront and one 16-byte vector per lane (1 KiB per block), the
        // shape that measures fastest on large messages (bounded below by 1 block)
        int threads = o.threads ? o.threads : 64;
        const size_t per_block = (size_t)threads * 16;
        long blocks = o.blocks ? o.blocks : (long)((bytes + per_block - 1) / per_block);
        if (blocks < 1) blocks = 1;
        if (blocks > (1 << 22)) blocks = 1 << 22;
        const double ms = time_ms([&] {
            return nvshmem_perftest_ring_rma(dst, src, bytes, (int)blocks, threads, o.scope, is_get ? 1 : 0, 1, nullptr);
        }, o.iters, o.warmup);
        gbs.push_back((double)bytes / ms / 1e6);  // payload of one PE, as the reference reports it
    }
    print_table(is_get ? "shmem_get_bw" : "shmem_put_bw", scope_name(o.scope), "BW", "GB/s per PE", sizes, gbs);
    printf("# %d PEs move that payload at once: aggregate payload = npes x BW, HBM traffic = 2 x that\n", o.npes);
    nvshmem_free(src);
    nvshmem_free(dst);
    return 0;
}

// shmem_p_bw / shmem_g_bw / shmem_st_bw / shmem_atomic_bw: size = bytes one PE moves per launch
int run_element(const Options &o, int what) {
    static const char *jobs[] = {"shmem_p_bw", "shmem_g_bw", "shmem_st_bw", "shmem_atomic_bw"};
    void *src = nvshmem_malloc(o.max_bytes), *dst = nvshmem_malloc(o.max_bytes);
    if (!src || !dst) return 1;
    std::vector<size_t> sizes = sweep(o, (size_t)o.elem);
    std::vector<double> gbs;
    for (size_t bytes : sizes) {
        const size_t nelems = bytes / (size_t)o.elem;
        // default: 256 threads, four elements per thread, at most 2^20 blocks per PE
        const int threads = o.threads ? o.threads : 256;
        long blocks = o.blocks ? o.blocks : (long)((nelems + 4 * (size_t)threads - 1) / (4 * (size_t)threads));
        if (blocks < 1) blocks = 1;
        if (blocks > (1 << 20)) blocks = 1 << 20;
        const double ms = time_ms([&] {
            return nvshmem_perftest_element_bw(what, o.elem, dst, src, nelems, (int)blocks, threads, nullptr);
        }, o.iters, o.warmup);
        gbs.push_back((double)bytes / ms / 1e6);
    }
    char scope[32];
    snprintf(scope, sizeof scope, "%d-byte", o.elem);
    print_table(jobs[what], scope, "BW", "GB/s per PE", sizes, gbs);
    printf("# %d PEs move that payload at once: aggregate payload = npes x BW\n", o.npes);
    nvshmem_free(src);
    nvshmem_free(dst);
    return 0;
}

enum { kReduce, kReducescatter, kFcollect, kAlltoall, kBroadcast };

int run_host_collective(const Options &o, int what) {
    const size_t n = (size_t)o.npes;
    // bytes = what one PE contributes; the larger of source and dest per PE is npes times that
    void *src = nvshmem_malloc(o.max_bytes * n), *dst = nvshmem_malloc(o.max_bytes * n);
    if (!src || !dst) return 1;
    std::vector<size_t> sizes = sweep(o, 4);
    std::vector<double> us, gbs;
    hipStream_t stream = nullptr;
    if (o.graph) CHECK_HIP(hipStreamCreate(&stream));
    for (size_t bytes : sizes) {
        double alg = 0;
        auto call = [&]() -> int {
            switch (what) {
                case kReduce:
                    alg = 2.0 * n * bytes;
                    return nvshmemx_float_sum_reduce_on_stream(NVSHMEM_TEAM_WORLD, (float *)dst, (const float *)src, bytes / 4, stream);
                case kReducescatter:  // every PE holds npes blocks of `bytes`
                    alg = (double)(n + 1) * n * bytes;
                    return nvshmemx_float_sum_reducescatter_on_stream(NVSHMEM_TEAM_WORLD, (float *)dst, (const float *)src, bytes / 4, stream);
                case kFcollect:
                    alg = (double)(n + 1) * n * bytes;
                    return nvshmemx_fcollectmem_on_stream(NVSHMEM_TEAM_WORLD, dst, src, bytes, stream);
                case kAlltoall:  // `bytes` per destination
                    alg = 2.0 * n * n * bytes;
                    return nvshmemx_alltoallmem_on_stream(NVSHMEM_TEAM_WORLD, dst, src, bytes, stream);
                default:
                    alg = (double)(n + 1) * bytes;
                    return nvshmemx_broadcastmem_on_stream(NVSHMEM_TEAM_WORLD, dst, src, bytes, 0, stream);
            }
        };
        const double ms = o.graph ? time_graph_ms(call, o.iters, stream) : time_ms(call, o.iters, o.warmup);
        us.push_back(ms * 1e3);
        gbs.push_back(alg / ms / 1e6);
    }
    static const char *names[] = {"reduction_on_stream", "reducescatter_on_stream", "fcollect_on_stream",
                                  "alltoall_on_stream", "bcast_on_stream"};
    print_table(names[what], o.graph ? "graph" : "stream", "latency", "us", sizes, us);
    print_table(names[what], o.graph ? "graph" : "stream", "algorithmic BW", "GB/s", sizes, gbs);
    if (stream) CHECK_HIP(hipStreamDestroy(stream));
    nvshmem_free(src);
    nvshmem_free(dst);
    return 0;
}

int run_device_latency(const Options &o, bool barrier_only, bool sync = false) {
    const size_t n = (size_t)o.npes;
    const size_t cap = barrier_only ? 64 : o.max_bytes;
    void *src = nvshmem_malloc(cap * n), *dst = nvshmem_malloc(cap * n);
    if (!src || !dst) return 1;
    const int threads = o.threads ? o.threads : 256;
    // per-call time = (launch with K + 1 calls - launch with 1 call) / K: the launch is paid once
    auto latency_us = [&](int what, size_t count) {
        auto one = [&] { return nvshmem_perftest_device_team_coll_loop(what, NVSHMEM_TEAM_WORLD, dst, src, count, 0, 1, o.scope, threads, nullptr); };
        auto many = [&] { return nvshmem_perftest_device_team_coll_loop(what, NVSHMEM_TEAM_WORLD, dst, src, count, 0, o.iters + 1, o.scope, threads, nullptr); };
        const double t1 = time_ms(one, 5, 2), tk = time_ms(many, 5, 2);
        return (tk - t1) * 1e3 / o.iters;
    };
    if (barrier_only) {
        printf("#%s\n%-8s  %-16s\n%-8s  %-16.6f\n", sync ? "sync_latency" : "barrier_latency", "scope", "latency (us)",
               scope_name(o.scope), latency_us(sync ? 6 : 5, 0));
    } else {
        std::vector<size_t> sizes = sweep(o, 4);
        static const struct { int what; const char *job; } calls[] = {
            {0, "reduction_latency"}, {1, "reducescatter_latency"}, {2, "fcollect_latency"},
            {3, "alltoall_latency"}, {4, "bcast_latency"}};
        for (const auto &c : calls) {
            std::vector<double> us;
            for (size_t bytes : sizes) us.push_back(latency_us(c.what, c.what <= 1 ? bytes / 4 : bytes));
            print_table(c.job, scope_name(o.scope), "latency", "us", sizes, us);
        }
        // (value, location) maximum of one pair per PE, block scope (redmaxloc_latency.cu)
        auto maxloc = [&](int k) { return nvshmem_perftest_device_maxloc(NVSHMEM_TEAM_WORLD, dst, src, 1, k, threads, nullptr, nullptr); };
        const double t1 = time_ms([&] { return maxloc(1); }, 5, 2), tk = time_ms([&] { return maxloc(o.iters + 1); }, 5, 2);
        printf("#redmaxloc_latency\n%-10s  %-8s  %-16s\n%-10d  %-8s  %-16.6f\n", "size(B)", "scope", "latency (us)", 16,
               "block", (tk - t1) * 1e3 / o.iters);
    }
    nvshmem_free(src);
    nvshmem_free(dst);
    return 0;
}

// host-initiated transfers on the default stream between PE 0 and PE 1
int run_host_rma(const Options &o, bool is_get) {
    void *src = nvshmem_malloc(o.max_bytes), *dst = nvshmem_malloc(o.max_bytes);
    if (!src || !dst) return 1;
    std::vector<size_t> sizes = sweep(o, 1);
    std::vector<double> gbs, us;
    for (size_t bytes : sizes) {
        const double ms = time_ms([&] {
            if (is_get) nvshmemx_getmem_on_stream(dst, src, bytes, 1, nullptr);
            else nvshmemx_putmem_on_stream(dst, src, bytes, 1, nullptr);
            return 0;
        }, o.iters, o.warmup);
        gbs.push_back((double)bytes / ms / 1e6);
        us.push_back(ms * 1e3);
    }
    print_table(is_get ? "get_on_stream" : "put_on_stream", "stream", "latency", "us", sizes, us);
    print_table(is_get ? "get_on_stream" : "put_on_stream", "stream", "BW", "GB/s payload", sizes, gbs);
    nvshmem_free(src);
    nvshmem_free(dst);
    return 0;
}

// barrier_all_on_stream.cpp / barrier_on_stream.cpp / sync_all_on_stream.cpp / sync_on_stream.cpp:
// microseconds per call, calls queued back to back on the default stream
int run_host_sync(const Options &o, bool sync) {
    const double all = time_ms([&] {
        if (sync) nvshmemx_sync_all_on_stream(nullptr); else nvshmemx_barrier_all_on_stream(nullptr);
        return 0;
    }, o.iters, o.warmup);
    const double team = time_ms([&] {
        return sync ? nvshmemx_team_sync_on_stream(NVSHMEM_TEAM_WORLD, nullptr)
                    : nvshmemx_barrier_on_stream(NVSHMEM_TEAM_WORLD, nullptr);
    }, o.iters, o.warmup);
    printf("#%s\n%-8s  %-16s\n%-8s  %-16.6f\n", sync ? "sync_all_on_stream" : "barrier_all_on_stream", "scope",
           "latency (us)", "stream", all * 1e3);
    printf("#%s\n%-8s  %-16s\n%-8s  %-16.6f\n", sync ? "sync_on_stream" : "barrier_on_stream", "scope",
           "latency (us)", "stream", team * 1e3);
    return 0;
}

// perftest/host/init/malloc.cpp: allocations of doubling size until the heap is full, then all
// freed; microseconds of host time per call (the allocator touches no device memory)
int run_malloc(const Options &o) {
    std::vector<void *> held;
    std::vector<size_t> sizes;
    std::vector<double> alloc_us, free_us;
    for (size_t bytes = o.min_bytes; bytes <= o.max_bytes; bytes *= 2) {
        timespec a, b;
        clock_gettime(CLOCK_MONOTONIC, &a);
        void *p = nvshmem_malloc(bytes);
        clock_gettime(CLOCK_MONOTONIC, &b);
        if (!p) break;
        held.push_back(p);
        sizes.push_back(bytes);
        alloc_us.push_back((b.tv_sec - a.tv_sec) * 1e6 + (b.tv_nsec - a.tv_nsec) * 1e-3);
    }
    for (void *p : held) {
        timespec a, b;
        clock_gettime(CLOCK_MONOTONIC, &a);
        nvshmem_free(p);
        clock_gettime(CLOCK_MONOTONIC, &b);
        free_us.push_back((b.tv_sec - a.tv_sec) * 1e6 + (b.tv_nsec - a.tv_nsec) * 1e-3);
    }
    print_table("nvshmem_malloc", "host", "latency", "us", sizes, alloc_us);
    print_table("nvshmem_free", "host", "latency", "us", sizes, free_us);
    return sizes.empty() ? 1 : 0;
}

// (launch with K + 1 repetitions - launch with 1) / K, like run_device_latency; sig is cleared before
// every launch because the ping-pong kinds count from zero.
int run_pt2pt_latency(const Options &o) {
    void *data = nvshmem_malloc(o.max_bytes);
    uint64_t *sig = (uint64_t *)nvshmem_calloc(2, sizeof(uint64_t));
    if (!data || !sig) return 1;
    const int threads = o.threads ? o.threads : 256;
    auto clear = [&] {
        for (int pe = 0; pe < 2; ++pe) CHECK_HIP(hipMemsetAsync(nvshmem_ptr(sig, pe), 0, 16, nullptr));
    };
    auto latency_us = [&](auto launch) {
        auto one = [&] { clear(); return launch(1); };
        auto many = [&] { clear(); return launch(o.iters + 1); };
        const double t1 = time_ms(one, 5, 2), tk = time_ms(many, 5, 2);
        return (tk - t1) * 1e3 / o.iters;
    };
    std::vector<size_t> sizes = sweep(o, 1);
    static const struct { int what; const char *job; } sized[] = {
        {NVSHMEM_PERFTEST_LAT_PUT, "shmem_put_latency"}, {NVSHMEM_PERFTEST_LAT_GET, "shmem_get_latency"}};
    for (const auto &c : sized) {
        std::vector<double> us;
        for (size_t bytes : sizes)
            us.push_back(latency_us([&](int k) { return nvshmem_perftest_pt2pt_latency(c.what, data, sig, bytes, k, threads, nullptr); }));
        print_table(c.job, "block", "latency", "us", sizes, us);
    }
    {
        std::vector<double> us;  // a full round trip, as the reference reports it
        for (size_t bytes : sizes)
            us.push_back(latency_us([&](int k) { return nvshmem_perftest_put_signal_pingpong(data, sig, bytes, k, threads, nullptr); }));
        print_table("shmem_put_signal_ping_pong_latency", "block", "round trip", "us", sizes, us);
    }
    static const struct { int what; const char *job; } scalar[] = {
        {NVSHMEM_PERFTEST_LAT_P, "shmem_p_latency (p + quiet)"},
        {NVSHMEM_PERFTEST_LAT_G, "shmem_g_latency"},
        {NVSHMEM_PERFTEST_LAT_ATOMIC, "shmem_atomic_latency (fetch_add)"},
        {NVSHMEM_PERFTEST_LAT_SIGNAL_PINGPONG, "shmem_signal_ping_pong_latency (round trip)"},
        {NVSHMEM_PERFTEST_LAT_P_PINGPONG, "shmem_p_ping_pong_latency (round trip)"},
        {NVSHMEM_PERFTEST_LAT_ATOMIC_PINGPONG, "shmem_atomic_ping_pong_latency (round trip)"}};
    printf("#scalar operations, PE 0 <-> PE 1\n%-48s  %-16s\n", "test", "latency (us)");
    for (const auto &c : scalar)
        printf("%-48s  %-16.6f\n", c.job,
               latency_us([&](int k) { return nvshmem_perftest_pt2pt_latency(c.what, data, sig, 8, k, threads, nullptr); }));
    nvshmem_free(data);
    nvshmem_free(sig);
    return 0;
}

}  // namespace

int main(int argc, char **argv) {
    const Options o = parse(argc, argv);
    const bool device_lat = o.test == "coll_latency" || o.test == "barrier_latency" || o.test == "sync_latency" ||
                            o.test == "pt2pt_latency" || o.test == "barrier_on_stream" || o.test == "sync_on_stream";
    // heap: source and dest of the largest size, times npes for the collectives
    const bool rma = o.test == "put_bw" || o.test == "get_bw" || o.test == "pt2pt_latency" || o.test == "p_bw" ||
                     o.test == "g_bw" || o.test == "st_bw" || o.test == "atomic_bw" || o.test == "malloc" ||
                     o.test == "host_put_bw" || o.test == "host_get_bw";
    Options eff = o;
    if (device_lat && o.max_bytes > ((size_t)1 << 20)) eff.max_bytes = (size_t)1 << 20;
    const size_t per_pe = (rma ? 2 * eff.max_bytes : 2 * eff.max_bytes * (size_t)eff.npes) + ((size_t)16 << 20);
    if (nvshmemx_amd_init(eff.npes, per_pe) != 0) {
        fprintf(stderr, "nvshmem_perftest: init failed: %s\n", nvshmemx_amd_last_error());
        return 1;
    }
    int rc;
    if (o.test == "put_bw") rc = run_rma(eff, false);
    else if (o.test == "get_bw") rc = run_rma(eff, true);
    else if (o.test == "p_bw") rc = run_element(eff, NVSHMEM_PERFTEST_ELEMENT_P);
    else if (o.test == "g_bw") rc = run_element(eff, NVSHMEM_PERFTEST_ELEMENT_G);
    else if (o.test == "st_bw") rc = run_element(eff, NVSHMEM_PERFTEST_ELEMENT_ST);
    else if (o.test == "atomic_bw") rc = run_element(eff, NVSHMEM_PERFTEST_ELEMENT_ADD);
    else if (o.test == "reduce") rc = run_host_collective(eff, kReduce);
    else if (o.test == "reducescatter") rc = run_host_collective(eff, kReducescatter);
    else if (o.test == "fcollect") rc = run_host_collective(eff, kFcollect);
    else if (o.test == "alltoall") rc = run_host_collective(eff, kAlltoall);
    else if (o.test == "broadcast") rc = run_host_collective(eff, kBroadcast);
    else if (o.test == "coll_latency") rc = run_device_latency(eff, false);
    else if (o.test == "barrier_latency") rc = run_device_latency(eff, true);
    else if (o.test == "sync_latency") rc = run_device_latency(eff, true, true);
    else if (o.test == "barrier_on_stream") rc = run_host_sync(eff, false);
    else if (o.test == "sync_on_stream") rc = run_host_sync(eff, true);
    else if (o.test == "malloc") rc = run_malloc(eff);
    else if (o.test == "pt2pt_latency") rc = run_pt2pt_latency(eff);
    else if (o.test == "host_put_bw") rc = run_host_rma(eff, false);
    else if (o.test == "host_get_bw") rc = run_host_rma(eff, true);
    else usage("unknown test");
    if (rc != 0) fprintf(stderr, "nvshmem_perftest: %s\n", nvshmemx_amd_last_error());
    nvshmem_finalize();
    return rc;
}
