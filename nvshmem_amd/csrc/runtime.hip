// Host runtime of the logical-PE NVSHMEM build: bring-up, symmetric heap, address translation,
// host-initiated RMA / signal operations on a stream, and the cooperative launcher.
//
// Reference counterparts: src/host/init/init.cu (state upload :146-197), src/host/mem/mem_heap.cpp
// (:2288-2387 public heap calls), src/host/comm/putget.cpp (:48-185 on-stream RMA),
// src/host/comm/sync.cpp (:60-115 on-stream signal ops),
// src/device/launch/collective_launch.cpp (:72-260).
#include "runtime.hpp"

#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "nvshmem.h"

namespace nvshmem_amd {

Runtime &Runtime::get() {
    static Runtime *rt = new Runtime();  // never destroyed: registrars of other libraries may
    return *rt;                          // still call in during process teardown
}

static thread_local std::string g_last_error;

void set_error(const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    fprintf(stderr, "nvshmem_amd: %s\n", buf);
}
void clear_error() { g_last_error.clear(); }

void refresh_symbols(Runtime &rt, bool force) {
    if (!rt.initialized || (!force && !rt.symbols_stale)) return;
    for (nvshmemi_amd_state_updater_t push : rt.updaters) {
        if (push(&rt.dev) != (int)hipSuccess) {
            (void)hipGetLastError();
            set_error("could not refresh a translation unit's device state block");
        }
    }
    rt.symbols_stale = false;
}

bool check_symmetric_range(Runtime &rt, const char *what, const void *p, uint64_t bytes,
                           uint64_t *off) {
    if (!rt.offset_of(p, off)) {
        set_error("%s: %p is not a symmetric address", what, p);
        return false;
    }
    // the runtime's own words (barrier rows, epoch, timeout record) end every slice and are not the
    // caller's to address
    const uint64_t usable = rt.heap_size - NVSHMEMI_AMD_INTERNAL_BYTES;
    if (bytes > usable || *off + bytes > usable) {
        set_error("%s: range [%p, +%llu) leaves the PE's heap slice (%llu bytes per PE)", what, p,
                  (unsigned long long)bytes, (unsigned long long)usable);
        return false;
    }
    return true;
}

uint64_t report_timeouts(Runtime &rt, const char *where) {
    if (!rt.initialized || !rt.dev.runtime_words) return 0;
    // callers have synchronised with the device: what a kernel stored to the pinned word has arrived
    if (rt.timeout_flag) {
        const uint64_t flag = __atomic_load_n(rt.timeout_flag, __ATOMIC_ACQUIRE);
        if (flag == rt.timeout_flag_seen) return 0;
        rt.timeout_flag_seen = flag;
    }
    uint64_t count = 0;
    if (hipMemcpy(&count, rt.dev.runtime_words + NVSHMEMI_AMD_TIMEOUT_COUNT_WORD, sizeof count,
                  hipMemcpyDeviceToHost) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    if (count <= rt.timeouts_seen) return 0;
    const uint64_t fresh = count - rt.timeouts_seen;
    rt.timeouts_seen = count;
    // Where: the newest record among the PEs' whose number lies in this period (a record's first word is the
    // timeout's number in the count; a PE keeps its latest one until nvshmemx_amd_read_timeout clears it).
    const uint64_t period_start = count - fresh;
    uint64_t rec[4] = {0, 0, 0, 0};
    int pe_hit = -1;
    uint64_t off = 0;
    rt.offset_of(rt.dev.timeout_record, &off);
    for (int pe = 0; pe < rt.npes; ++pe) {
        uint64_t r[4] = {0, 0, 0, 0};
        if (hipMemcpy(r, rt.slice(pe) + off, sizeof r, hipMemcpyDeviceToHost) != hipSuccess) continue;
        if (r[0] > period_start && r[0] > rec[0]) {
            pe_hit = pe;
            for (int i = 0; i < 4; ++i) rec[i] = r[i];
        }
    }
    (void)hipGetLastError();
    char where_text[160] = "";
    if (pe_hit >= 0)
        snprintf(where_text, sizeof where_text, "; e.g. PE %d waited at %p for %llu and last saw %llu", pe_hit,
                 (void *)(uintptr_t)rec[1], (unsigned long long)rec[3], (unsigned long long)rec[2]);
    set_error("%s: %llu device-side wait%s gave up after the spin limit of %llu polls (NVSHMEM_AMD_SPIN_LIMIT; 0 waits "
              "forever) and the kernel went on as if satisfied - results may be incomplete%s",
              where, (unsigned long long)fresh, fresh == 1 ? "" : "s", (unsigned long long)rt.dev.spin_limit, where_text);
    return fresh;
}

namespace {

bool require_init(Runtime &rt, const char *what) {
    if (rt.initialized) return true;
    set_error("%s called before nvshmem_init", what);
    return false;
}

uint64_t env_size(const char *name, uint64_t dflt) {
    const char *v = getenv(name);
    if (!v || !*v) return dflt;
    char *end = nullptr;
    double x = strtod(v, &end);
    if (end == v || x < 0) return dflt;
    switch (*end) {
        case 'k': case 'K': x *= 1024.0; break;
        case 'm': case 'M': x *= 1024.0 * 1024.0; break;
        case 'g': case 'G': x *= 1024.0 * 1024.0 * 1024.0; break;
        case 't': case 'T': x *= 1024.0 * 1024.0 * 1024.0 * 1024.0; break;
        default: break;
    }
    return (uint64_t)x;
}

__global__ void signal_op_kernel(uint64_t *sig_addr, uint64_t signal, int sig_op, int pe) {
    nvshmemi_signal_op_release(sig_addr, signal, sig_op, pe);
}

__global__ void signal_wait_kernel(uint64_t *sig_addr, int cmp, uint64_t cmp_value) {
    nvshmemi_wait_until<uint64_t>(sig_addr, cmp, cmp_value);
}

}  // namespace
}  // namespace nvshmem_amd

using namespace nvshmem_amd;

extern "C" {

const char *nvshmemx_amd_last_error(void) { return g_last_error.c_str(); }

void nvshmemi_amd_register_state_updater(nvshmemi_amd_state_updater_t fn) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    rt.updaters.insert(fn);
    rt.symbols_stale = true;  // pushed at the next library call, once the unit's code is loaded
}

void nvshmemi_amd_unregister_state_updater(nvshmemi_amd_state_updater_t fn) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    rt.updaters.erase(fn);
}

int nvshmemx_amd_module_init(void) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!rt.initialized) return NVSHMEMX_ERROR_INVALID_VALUE;
    refresh_symbols(rt, false);  // a no-op unless a unit registered since the last push
    return NVSHMEMX_SUCCESS;
}

int nvshmemx_amd_init(int npes, size_t symmetric_size) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    clear_error();
    if (rt.initialized) {
        set_error("nvshmemx_amd_init: already initialised (%d PEs); call nvshmem_finalize first",
                  rt.npes);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    if (npes < 1 || npes > NVSHMEMI_AMD_MAX_PES) {
        set_error("nvshmemx_amd_init: npes=%d outside [1, %d]", npes, NVSHMEMI_AMD_MAX_PES);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    const uint64_t min_slice = 1ull << 16;
    uint64_t want = symmetric_size < min_slice ? min_slice : (uint64_t)symmetric_size;
    // room for the runtime's own symmetric words (barrier row, epoch, timeout record)
    want += NVSHMEMI_AMD_INTERNAL_BYTES;
    // The distance between slices is the size asked for rounded up to 16 MiB (2 MiB for small heaps),
    // not to a power of two.  16 MiB multiples measured best for kernels that store one piece into
    // many slices at equal offsets (fcollect of 16 x 16 MiB: 6.0-6.2 TB/s against 5.2-5.6 at distances
    // that are odd multiples of 2 MiB); the copy engine and the reductions do not care.
    if (want > (1ull << 40)) {
        set_error("nvshmemx_amd_init: symmetric size %zu too large", symmetric_size);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    const uint64_t granule = want > (16ull << 20) ? (16ull << 20) : (2ull << 20);
    const uint64_t slice_bytes = (want + granule - 1) / granule * granule;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        set_error("nvshmemx_amd_init: no HIP device available");
        return NVSHMEMX_ERROR_GPU_NOT_SELECTED;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        set_error("nvshmemx_amd_init: hipGetDeviceProperties failed");
        return NVSHMEMX_ERROR_INTERNAL;
    }
    const uint64_t total = (uint64_t)npes * slice_bytes;
    // (the device code's division-free slice index is exact up to this size)
    if (total > (1ull << 39)) {
        set_error("nvshmemx_amd_init: %d PEs x %llu bytes exceed 512 GiB", npes, (unsigned long long)slice_bytes);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    void *mem = nullptr;
    hipError_t e = hipMalloc(&mem, total);
    if (e != hipSuccess || !mem) {
        (void)hipGetLastError();
        set_error("nvshmemx_amd_init: hipMalloc of %llu bytes (%d PEs x %llu) failed: %s",
                  (unsigned long long)total, npes, (unsigned long long)slice_bytes, hipGetErrorString(e));
        return NVSHMEMX_ERROR_OUT_OF_MEMORY;
    }
    rt.device = dev;
    rt.num_cus = prop.multiProcessorCount;
    rt.npes = npes;
    rt.heap_size = slice_bytes;
    rt.base = (char *)mem;
    // The runtime's own symmetric words (barrier row, epoch, timeout record) live in the last
    // granules of every slice, outside the allocator's space, so that user allocations start at the
    // slice base: large buffers then sit on the 1 KiB boundaries the streaming kernels like.
    const uint64_t internal_bytes = NVSHMEMI_AMD_INTERNAL_BYTES;
    rt.space.reset(new SymmetricSpace((uint64_t)(uintptr_t)rt.base, rt.heap_size - internal_bytes));
    rt.initialized = true;
    const uint64_t internal = (uint64_t)(uintptr_t)rt.base + rt.heap_size - internal_bytes;
    const uint64_t flags = internal;
    const uint64_t epoch = internal + NVSHMEMI_AMD_MAX_PES * sizeof(uint64_t);
    const uint64_t trec = epoch + NVSHMEMI_MALLOC_ALIGNMENT;
    for (int pe = 0; pe < npes; ++pe)
        NVSHMEM_AMD_HIP_CHECK(hipMemset(rt.slice(pe) + rt.heap_size - internal_bytes, 0, internal_bytes));

    memset(&rt.dev, 0, sizeof rt.dev);
    rt.dev.version = (1u << 16) + (uint32_t)sizeof(nvshmemi_device_state_t);
    rt.dev.mype = 0;
    rt.dev.npes = npes;
    rt.dev.heap_base = rt.base;
    rt.dev.heap_size = rt.heap_size;
    rt.dev.sync_flags = (uint64_t *)(uintptr_t)flags;
    rt.dev.sync_epoch = (uint64_t *)(uintptr_t)epoch;
    rt.dev.timeout_record = (uint64_t *)(uintptr_t)trec;
    rt.dev.runtime_words = (uint64_t *)(uintptr_t)(trec + NVSHMEMI_MALLOC_ALIGNMENT);
    void *flag = nullptr;
    if (hipHostMalloc(&flag, sizeof(uint64_t), hipHostMallocDefault) == hipSuccess && flag) {
        rt.timeout_flag = (uint64_t *)flag;
        *rt.timeout_flag = 0;
    } else {
        (void)hipGetLastError();  // without the word every report fetches the count from the GPU
        rt.timeout_flag = nullptr;
    }
    rt.timeout_flag_seen = 0;
    rt.dev.timeout_flag = rt.timeout_flag;
    rt.dev.spin_limit = env_size("NVSHMEM_AMD_SPIN_LIMIT", 1ull << 22);
    rt.dev.options = 0;
    if (const char *order = getenv("NVSHMEM_AMD_PUT_SIGNAL_ORDER")) {
        if (!strcmp(order, "payload")) rt.dev.options |= NVSHMEMI_AMD_OPTION_PUT_SIGNAL_PAYLOAD_ONLY;
        else if (strcmp(order, "full") && *order)
            fprintf(stderr, "nvshmem_amd: NVSHMEM_AMD_PUT_SIGNAL_ORDER=%s is neither \"payload\" nor \"full\"; "
                            "using full\n", order);
    }
    rt.dev.heap_magic = (1ull << 40) / (rt.heap_size >> 21) + 1;
    rt.plain_collective_launch = env_size("NVSHMEM_AMD_PLAIN_COLLECTIVE_LAUNCH", 0) != 0;
    rt.cacheable_source_bytes = env_size("NVSHMEM_AMD_CACHEABLE_SOURCE_BYTES", (size_t)256 << 20);
    rt.chunked_copy_bytes = env_size("NVSHMEM_AMD_CHUNKED_COPY_BYTES", (size_t)128 << 20);
    rt.lds_reduce_bytes = env_size("NVSHMEM_AMD_LDS_REDUCE_BYTES", (size_t)64 << 20);
    rt.two_step_reduce_members = (unsigned)env_size("NVSHMEM_AMD_TWO_STEP_REDUCE_MEMBERS", 16);
    rt.two_step_reduce_bytes = env_size("NVSHMEM_AMD_TWO_STEP_REDUCE_BYTES", (size_t)512 << 20);
    if (!teams_init(rt)) {
        teams_finalize(rt);
        (void)hipFree(rt.base);
        if (rt.timeout_flag) (void)hipHostFree(rt.timeout_flag);
        rt.timeout_flag = nullptr;
        rt.space.reset();
        rt.base = nullptr;
        rt.initialized = false;
        rt.npes = 0;
        return NVSHMEMX_ERROR_OUT_OF_MEMORY;
    }
    NVSHMEM_AMD_HIP_CHECK(hipDeviceSynchronize());
    refresh_symbols(rt, true);
    return NVSHMEMX_SUCCESS;
}

void nvshmem_init(void) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (rt.initialized) return;
    const int npes = (int)env_size("NVSHMEM_AMD_NPES", 8);
    const uint64_t size = env_size("NVSHMEM_SYMMETRIC_SIZE", 1ull << 30);
    if (nvshmemx_amd_init(npes, size) != NVSHMEMX_SUCCESS) {
        // reference: init failure ends the program (NVSHMEMI_CHECK_INIT / NONZERO_EXIT,
        // src/include/host/nvshmem_api.h:40-48)
        fprintf(stderr, "nvshmem_init failed: %s\n", nvshmemx_amd_last_error());
        exit(-1);
    }
}

void nvshmem_finalize(void) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!rt.initialized) return;
    (void)hipDeviceSynchronize();
    (void)report_timeouts(rt, "nvshmem_finalize");
    rt.timeouts_seen = 0;
    teams_finalize(rt);
    (void)hipFree(rt.base);
    if (rt.timeout_flag) (void)hipHostFree(rt.timeout_flag);
    rt.timeout_flag = nullptr;
    rt.timeout_flag_seen = 0;
    rt.space.reset();
    rt.base = nullptr;
    rt.initialized = false;
    rt.npes = 0;
    memset(&rt.dev, 0, sizeof rt.dev);
}

int nvshmemx_init_status(void) {
    return Runtime::get().initialized ? NVSHMEM_STATUS_IS_INITIALIZED
                                      : NVSHMEM_STATUS_NOT_INITIALIZED;
}

int nvshmem_init_thread(int requested, int *provided) {
    (void)requested;
    nvshmem_init();
    if (provided) *provided = NVSHMEM_THREAD_SERIALIZED;
    return 0;
}
void nvshmem_query_thread(int *provided) {
    if (provided) *provided = NVSHMEM_THREAD_SERIALIZED;
}
void nvshmem_global_exit(int status) {
    nvshmem_finalize();
    exit(status);
}
int nvshmemx_buffer_register(void *addr, size_t length) {
    if (!addr || length == 0) {
        set_error("nvshmemx_buffer_register: null buffer or zero length");
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    return 0;
}
int nvshmemx_buffer_unregister(void *addr) { return addr ? 0 : NVSHMEMX_ERROR_INVALID_VALUE; }
void nvshmemx_buffer_unregister_all(void) {}

int nvshmem_my_pe(void) { return 0; }
int nvshmem_n_pes(void) { return Runtime::get().npes; }
void nvshmem_info_get_version(int *major, int *minor) {
    if (major) *major = NVSHMEM_MAJOR_VERSION;
    if (minor) *minor = NVSHMEM_MINOR_VERSION;
}
void nvshmem_info_get_name(char *name) {
    if (name) snprintf(name, NVSHMEM_MAX_NAME_LEN, "%s", NVSHMEM_VENDOR_STRING);
}
void nvshmemx_vendor_get_version_info(int *major, int *minor, int *patch) {
    if (major) *major = NVSHMEM_VENDOR_MAJOR_VERSION;
    if (minor) *minor = NVSHMEM_VENDOR_MINOR_VERSION;
    if (patch) *patch = NVSHMEM_VENDOR_PATCH_VERSION;
}

void nvshmemx_amd_set_put_signal_order(int payload_only) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (payload_only) rt.dev.options |= NVSHMEMI_AMD_OPTION_PUT_SIGNAL_PAYLOAD_ONLY;
    else rt.dev.options &= ~NVSHMEMI_AMD_OPTION_PUT_SIGNAL_PAYLOAD_ONLY;
    if (rt.initialized) {
        NVSHMEM_AMD_HIP_CHECK(hipDeviceSynchronize());
        refresh_symbols(rt, true);
    }
}

int nvshmemx_amd_get_put_signal_order(void) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    return (rt.dev.options & NVSHMEMI_AMD_OPTION_PUT_SIGNAL_PAYLOAD_ONLY) ? 1 : 0;
}

void nvshmemx_amd_set_spin_limit(uint64_t polls) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    rt.dev.spin_limit = polls;
    if (rt.initialized) {
        NVSHMEM_AMD_HIP_CHECK(hipDeviceSynchronize());
        refresh_symbols(rt, true);
    }
}

uint64_t nvshmemx_amd_read_timeout(int pe, uint64_t out[4]) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    uint64_t rec[4] = {0, 0, 0, 0};
    if (!require_init(rt, "nvshmemx_amd_read_timeout") || pe < 0 || pe >= rt.npes) return 0;
    uint64_t off = 0;
    rt.offset_of(rt.dev.timeout_record, &off);
    NVSHMEM_AMD_HIP_CHECK(hipMemcpy(rec, rt.slice(pe) + off, sizeof rec, hipMemcpyDeviceToHost));
    NVSHMEM_AMD_HIP_CHECK(hipMemset(rt.slice(pe) + off, 0, sizeof rec));
    if (out) memcpy(out, rec, sizeof rec);
    return rec[0];
}

/* ---------------------------------------------------------------------------------------------
 * Symmetric heap.  One allocation decision serves every PE (same offset in every slice), which is
 * what the reference obtains by running the same allocator on every PE and checking symmetry.
 * Zero-size requests return NULL and free(NULL) does nothing, as in the reference
 * (NVSHMEMI_IS_NO_ACTION_BY_SIZE / _BY_PTR, mem_heap.cpp:2296, :2357).
 * ------------------------------------------------------------------------------------------- */
static void *heap_fail(Runtime &rt, const char *what, size_t size) {
    set_error("%s: could not allocate %zu bytes per PE from the symmetric heap (%llu bytes per PE, "
              "%llu free); raise NVSHMEM_SYMMETRIC_SIZE",
              what, size, (unsigned long long)rt.heap_size,
              (unsigned long long)rt.space->free_bytes());
    if (getenv("NVSHMEM_AMD_EXIT_ON_ERROR")) exit(-1);  // the reference always exits here
    return nullptr;
}

void *nvshmem_malloc(size_t size) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!require_init(rt, "nvshmem_malloc") || size == 0) return nullptr;
    refresh_symbols(rt, false);
    const uint64_t a = rt.space->allocate(size);
    if (!a) return heap_fail(rt, "nvshmem_malloc", size);
    return (void *)(uintptr_t)a;
}

void *nvshmem_calloc(size_t count, size_t size) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!require_init(rt, "nvshmem_calloc") || size == 0 || count == 0) return nullptr;
    refresh_symbols(rt, false);
    if (count > SIZE_MAX / size) return heap_fail(rt, "nvshmem_calloc", SIZE_MAX);
    const size_t bytes = count * size;
    const uint64_t a = rt.space->allocate(bytes);
    if (!a) return heap_fail(rt, "nvshmem_calloc", bytes);
    const uint64_t off = a - (uint64_t)(uintptr_t)rt.base;
    for (int pe = 0; pe < rt.npes; ++pe)
        NVSHMEM_AMD_HIP_CHECK(hipMemsetAsync(rt.slice(pe) + off, 0, bytes, nullptr));
    NVSHMEM_AMD_HIP_CHECK(hipStreamSynchronize(nullptr));
    return (void *)(uintptr_t)a;
}

void *nvshmem_align(size_t alignment, size_t size) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!require_init(rt, "nvshmem_align") || size == 0) return nullptr;
    refresh_symbols(rt, false);
    if (alignment == 0 || (alignment & (alignment - 1)) || alignment % sizeof(void *)) {
        set_error("nvshmem_align: alignment %zu is not a power of two multiple of %zu", alignment,
                  sizeof(void *));
        return nullptr;
    }
    const uint64_t a = rt.space->allocate_aligned(alignment, size);
    if (!a) return heap_fail(rt, "nvshmem_align", size);
    return (void *)(uintptr_t)a;
}

void nvshmem_free(void *ptr) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!ptr || !require_init(rt, "nvshmem_free")) return;
    // barrier before release, as in the reference: no PE may still be using the block
    NVSHMEM_AMD_HIP_CHECK(hipDeviceSynchronize());
    (void)report_timeouts(rt, "nvshmem_free");
    uint64_t off = 0;
    if (!rt.offset_of(ptr, &off) ||
        !rt.space->deallocate((uint64_t)(uintptr_t)rt.base + off)) {
        set_error("nvshmem_free: %p is not a live symmetric allocation", ptr);
        if (getenv("NVSHMEM_AMD_EXIT_ON_ERROR")) exit(-1);  // reference: custom_malloc.cpp:159-162
    }
}

void *nvshmem_ptr(const void *ptr, int pe) {
    Runtime &rt = Runtime::get();
    uint64_t off = 0;
    if (pe < 0 || pe >= rt.npes || !rt.offset_of(ptr, &off)) return nullptr;
    return rt.slice(pe) + off;
}

/* ---------------------------------------------------------------------------------------------
 * Ordering.  Every logical PE's work is stream work of this one process, so completion of all PEs
 * is completion of the device's streams.
 * ------------------------------------------------------------------------------------------- */
static uint64_t device_wait(const char *where) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    refresh_symbols(rt, false);
    NVSHMEM_AMD_HIP_CHECK(hipDeviceSynchronize());
    return report_timeouts(rt, where);
}
void nvshmem_quiet(void) { (void)device_wait("nvshmem_quiet"); }
void nvshmem_fence(void) { (void)device_wait("nvshmem_fence"); }
void nvshmem_barrier_all(void) { (void)device_wait("nvshmem_barrier_all"); }
uint64_t nvshmemx_amd_timeout_count(void) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    uint64_t count = 0;
    if (rt.initialized && rt.dev.runtime_words)
        NVSHMEM_AMD_HIP_CHECK(hipMemcpy(&count, rt.dev.runtime_words + NVSHMEMI_AMD_TIMEOUT_COUNT_WORD, sizeof count,
                                        hipMemcpyDeviceToHost));
    return count;
}
/* The host thread stands for every PE of any team, so a team barrier is the device-wide wait too. */
static int known_team(const char *what, nvshmem_team_t team) {
    TeamLaunch tl;
    return resolve_team(Runtime::get(), what, team, &tl) ? 0 : NVSHMEMX_ERROR_INVALID_VALUE;
}
int nvshmem_barrier(nvshmem_team_t team) {
    std::lock_guard<std::recursive_mutex> lock(Runtime::get().mu);
    if (known_team("nvshmem_barrier", team)) return NVSHMEMX_ERROR_INVALID_VALUE;
    return device_wait("nvshmem_barrier") ? NVSHMEMX_ERROR_INTERNAL : 0;
}
void nvshmem_sync_all(void) { nvshmem_barrier_all(); }
int nvshmem_team_sync(nvshmem_team_t team) { return nvshmem_barrier(team); }
/* Work of all PEs submitted to one stream is already ordered on it. */
void nvshmemx_barrier_all_on_stream(nvshmemx_stream_t) {}
int nvshmemx_barrier_on_stream(nvshmem_team_t team, nvshmemx_stream_t) {
    std::lock_guard<std::recursive_mutex> lock(Runtime::get().mu);
    return known_team("nvshmemx_barrier_on_stream", team);
}
void nvshmemx_sync_all_on_stream(nvshmemx_stream_t) {}
int nvshmemx_team_sync_on_stream(nvshmem_team_t team, nvshmemx_stream_t) {
    std::lock_guard<std::recursive_mutex> lock(Runtime::get().mu);
    return known_team("nvshmemx_team_sync_on_stream", team);
}
void nvshmemx_quiet_on_stream(nvshmemx_stream_t) {}

/* ---------------------------------------------------------------------------------------------
 * Host-initiated RMA: a device-to-device copy to/from the translated address, as the reference
 * does with cudaMemcpyAsync on its load/store path (putget.cpp:48-185).
 * ------------------------------------------------------------------------------------------- */
static bool rma_target(Runtime &rt, const char *what, const void *sym, size_t bytes, int pe,
                       char **out) {
    if (!require_init(rt, what)) return false;
    if (pe < 0 || pe >= rt.npes) {
        set_error("%s: pe %d outside [0, %d)", what, pe, rt.npes);
        return false;
    }
    uint64_t off = 0;
    if (!check_symmetric_range(rt, what, sym, bytes, &off)) return false;
    *out = rt.slice(pe) + off;
    return true;
}

/* Copies between device buffers that are too large for the Infinity Cache to absorb go through the
 * library's own copy engine, one wavefront per KiB: measured 6.8 TB/s (read + written) at 1 GiB against
 * 5.2 TB/s for hipMemcpyAsync, which is the faster one while source and destination fit the cache
 * together.  Anything else (host memory on either side, smaller sizes) is a hipMemcpyAsync. */
__global__ __launch_bounds__(64) void bulk_copy_kernel(char *dst, const char *src, size_t bytes) {
    const size_t at = (size_t)blockIdx.x * 1024;
    nvshmemi_memcpy_threadgroup<NVSHMEMI_THREADGROUP_BLOCK>(dst + at, src + at, bytes - at < 1024 ? bytes - at : 1024);
}

static bool on_this_device(const void *p) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();  // ordinary host memory is reported as an error
        return false;
    }
    return attr.type == hipMemoryTypeDevice;
}

static void stream_copy(char *dst, const char *src, size_t bytes, bool other_is_device,
                        hipStream_t stream) {
    constexpr size_t kBulk = (size_t)128 << 20;  // source + destination no longer fit the 256 MiB cache
    const size_t blocks = (bytes + 1023) / 1024;
    if (bytes > kBulk && blocks <= 0x7fffffffull && other_is_device) {
        hipLaunchKernelGGL(bulk_copy_kernel, dim3((unsigned)blocks), dim3(64), 0, stream, dst, src, bytes);
        NVSHMEM_AMD_HIP_CHECK(hipGetLastError());
        return;
    }
    NVSHMEM_AMD_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, stream));
}

void nvshmemx_putmem_on_stream(void *dest, const void *source, size_t bytes, int pe,
                               nvshmemx_stream_t stream) {
    Runtime &rt = Runtime::get();
    char *target = nullptr;
    if (bytes == 0 || !rma_target(rt, "nvshmemx_putmem_on_stream", dest, bytes, pe, &target)) return;
    stream_copy(target, (const char *)source, bytes, bytes > ((size_t)128 << 20) && on_this_device(source),
                (hipStream_t)stream);
}

void nvshmemx_getmem_on_stream(void *dest, const void *source, size_t bytes, int pe,
                               nvshmemx_stream_t stream) {
    Runtime &rt = Runtime::get();
    char *target = nullptr;
    if (bytes == 0 || !rma_target(rt, "nvshmemx_getmem_on_stream", source, bytes, pe, &target)) return;
    stream_copy((char *)dest, target, bytes, bytes > ((size_t)128 << 20) && on_this_device(dest),
                (hipStream_t)stream);
}

void nvshmemx_putmem_nbi_on_stream(void *dest, const void *source, size_t bytes, int pe,
                                   nvshmemx_stream_t stream) {
    nvshmemx_putmem_on_stream(dest, source, bytes, pe, stream);
}
void nvshmemx_getmem_nbi_on_stream(void *dest, const void *source, size_t bytes, int pe,
                                   nvshmemx_stream_t stream) {
    nvshmemx_getmem_on_stream(dest, source, bytes, pe, stream);
}
void nvshmem_putmem(void *dest, const void *source, size_t bytes, int pe) {
    nvshmemx_putmem_on_stream(dest, source, bytes, pe, nullptr);
    NVSHMEM_AMD_HIP_CHECK(hipStreamSynchronize(nullptr));
}
void nvshmem_getmem(void *dest, const void *source, size_t bytes, int pe) {
    nvshmemx_getmem_on_stream(dest, source, bytes, pe, nullptr);
    NVSHMEM_AMD_HIP_CHECK(hipStreamSynchronize(nullptr));
}
void nvshmem_putmem_nbi(void *dest, const void *source, size_t bytes, int pe) {
    nvshmemx_putmem_on_stream(dest, source, bytes, pe, nullptr);
}
void nvshmem_getmem_nbi(void *dest, const void *source, size_t bytes, int pe) {
    nvshmemx_getmem_on_stream(dest, source, bytes, pe, nullptr);
}

#define NVSHMEMI_DEFINE_TYPED_RMA_HOST(NAME, TYPE, TAG)                                          \
    void nvshmem_##NAME##_put(TYPE *dest, const TYPE *source, size_t nelems, int pe) {           \
        nvshmem_putmem(dest, source, nelems * sizeof(TYPE), pe);                                 \
    }                                                                                            \
    void nvshmem_##NAME##_get(TYPE *dest, const TYPE *source, size_t nelems, int pe) {           \
        nvshmem_getmem(dest, source, nelems * sizeof(TYPE), pe);                                 \
    }                                                                                            \
    void nvshmemx_##NAME##_put_on_stream(TYPE *dest, const TYPE *source, size_t nelems, int pe,  \
                                         nvshmemx_stream_t stream) {                             \
        nvshmemx_putmem_on_stream(dest, source, nelems * sizeof(TYPE), pe, stream);              \
    }                                                                                            \
    void nvshmemx_##NAME##_get_on_stream(TYPE *dest, const TYPE *source, size_t nelems, int pe,  \
                                         nvshmemx_stream_t stream) {                             \
        nvshmemx_getmem_on_stream(dest, source, nelems * sizeof(TYPE), pe, stream);              \
    }
NVSHMEMI_REPT_FOR_STANDARD_RMA_TYPES(NVSHMEMI_DEFINE_TYPED_RMA_HOST)
#undef NVSHMEMI_DEFINE_TYPED_RMA_HOST

void nvshmemx_signal_op_on_stream(uint64_t *sig_addr, uint64_t signal, int sig_op, int pe,
                                  nvshmemx_stream_t stream) {
    Runtime &rt = Runtime::get();
    char *target = nullptr;
    if (!rma_target(rt, "nvshmemx_signal_op_on_stream", sig_addr, sizeof(uint64_t), pe, &target))
        return;
    sig_op &= NVSHMEMI_AMD_SIGNAL_OP_MASK;  // an ordering hint means nothing here: stream order already orders
    if (sig_op != NVSHMEM_SIGNAL_SET && sig_op != NVSHMEM_SIGNAL_ADD) {
        set_error("nvshmemx_signal_op_on_stream: sig_op %d is neither SET (9) nor ADD (10)", sig_op);
        return;
    }
    {
        std::lock_guard<std::recursive_mutex> lock(rt.mu);
        refresh_symbols(rt, false);
    }
    hipLaunchKernelGGL(signal_op_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, sig_addr, signal,
                       sig_op, pe);
    NVSHMEM_AMD_HIP_CHECK(hipGetLastError());
}

void nvshmemx_signal_wait_until_on_stream(uint64_t *sig_addr, int cmp, uint64_t cmp_value,
                                          nvshmemx_stream_t stream) {
    Runtime &rt = Runtime::get();
    uint64_t off = 0;
    if (!require_init(rt, "nvshmemx_signal_wait_until_on_stream") ||
        !check_symmetric_range(rt, "nvshmemx_signal_wait_until_on_stream", sig_addr,
                               sizeof(uint64_t), &off))
        return;
    if (cmp < NVSHMEM_CMP_EQ || cmp > NVSHMEM_CMP_GE) {
        set_error("nvshmemx_signal_wait_until_on_stream: unknown comparison %d", cmp);
        return;
    }
    {
        std::lock_guard<std::recursive_mutex> lock(rt.mu);
        refresh_symbols(rt, false);
    }
    hipLaunchKernelGGL(signal_wait_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, sig_addr, cmp,
                       cmp_value);
    NVSHMEM_AMD_HIP_CHECK(hipGetLastError());
}

void nvshmemx_putmem_signal_on_stream(void *dest, const void *source, size_t bytes,
                                      uint64_t *sig_addr, uint64_t signal, int sig_op, int pe,
                                      nvshmemx_stream_t stream) {
    nvshmemx_putmem_on_stream(dest, source, bytes, pe, stream);
    nvshmemx_signal_op_on_stream(sig_addr, signal, sig_op, pe, stream);
}
void nvshmemx_putmem_signal_nbi_on_stream(void *dest, const void *source, size_t bytes,
                                          uint64_t *sig_addr, uint64_t signal, int sig_op, int pe,
                                          nvshmemx_stream_t stream) {
    nvshmemx_putmem_signal_on_stream(dest, source, bytes, sig_addr, signal, sig_op, pe, stream);
}

/* ---------------------------------------------------------------------------------------------
 * Cooperative launch of one grid that carries every logical PE in its z dimension.
 * ------------------------------------------------------------------------------------------- */
static int max_blocks_per_pe(Runtime &rt, const void *func, unsigned threads, size_t shared_mem,
                             int *out) {
    int per_cu = 0;
    hipError_t e =
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, func, (int)threads, shared_mem);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_error("collective launch: occupancy query failed: %s", hipGetErrorString(e));
        return NVSHMEMX_ERROR_COLLECTIVE_LAUNCH_FAILED;
    }
    *out = (int)(((long long)per_cu * rt.num_cus) / rt.npes);
    return NVSHMEMX_SUCCESS;
}

int nvshmemx_amd_collective_launch_query_gridsize(const void *func, unsigned block_x,
                                                  unsigned block_y, unsigned block_z,
                                                  size_t shared_mem, int *gridsize) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!require_init(rt, "nvshmemx_collective_launch_query_gridsize") || !gridsize)
        return NVSHMEMX_ERROR_INVALID_VALUE;
    return max_blocks_per_pe(rt, func, block_x * block_y * block_z, shared_mem, gridsize);
}

int nvshmemx_amd_collective_launch(const void *func, unsigned grid_x, unsigned grid_y,
                                   unsigned grid_z, unsigned block_x, unsigned block_y,
                                   unsigned block_z, void **args, size_t shared_mem,
                                   nvshmemx_stream_t stream) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!require_init(rt, "nvshmemx_collective_launch")) return NVSHMEMX_ERROR_INVALID_VALUE;
    refresh_symbols(rt, false);
    const unsigned threads = block_x * block_y * block_z;
    if (threads == 0 || threads > 1024) {
        set_error("collective launch: block of %u threads", threads);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    int cap = 0;
    int rc = max_blocks_per_pe(rt, func, threads, shared_mem, &cap);
    if (rc != NVSHMEMX_SUCCESS) return rc;
    if (grid_x == 0 && grid_y == 0 && grid_z == 0) {
        grid_x = (unsigned)cap;
        grid_y = 1;
        grid_z = 1;
    }
    if (grid_z != 1) {
        set_error("collective launch: grid.z must be 1 (the z dimension carries the PE index)");
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    const unsigned long long per_pe = (unsigned long long)grid_x * grid_y;
    if (per_pe == 0 || per_pe > (unsigned long long)cap) {
        set_error("collective launch: %llu blocks per PE x %d PEs cannot be co-resident "
                  "(limit %d blocks per PE for %u threads)",
                  per_pe, rt.npes, cap, threads);
        return NVSHMEMX_ERROR_COLLECTIVE_LAUNCH_FAILED;
    }
    // A cooperative launch guarantees that all blocks are resident together, whatever else runs on
    // the GPU, and costs about 20 us more than a plain launch here.  The grid has just been checked
    // against the occupancy limit, so a plain launch gives the same co-residency as long as no
    // other kernel holds compute units while waiting for this one: NVSHMEM_AMD_PLAIN_COLLECTIVE_
    // LAUNCH=1 opts into that for programs that launch their PE kernels one at a time.
    const dim3 grid(grid_x, grid_y, (unsigned)rt.npes), block(block_x, block_y, block_z);
    hipError_t e = rt.plain_collective_launch
                       ? hipLaunchKernel(func, grid, block, args, shared_mem, (hipStream_t)stream)
                       : hipLaunchCooperativeKernel(func, grid, block, args, (unsigned)shared_mem,
                                                    (hipStream_t)stream);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_error("collective launch: %s failed: %s",
                  rt.plain_collective_launch ? "hipLaunchKernel" : "hipLaunchCooperativeKernel",
                  hipGetErrorString(e));
        return NVSHMEMX_ERROR_COLLECTIVE_LAUNCH_FAILED;
    }
    return NVSHMEMX_SUCCESS;
}

/* ---------------------------------------------------------------------------------------------
 * Allocator exposed on its own (no GPU involved).
 * ------------------------------------------------------------------------------------------- */
struct nvshmemi_amd_mspace {
    SymmetricSpace space;
    nvshmemi_amd_mspace(uint64_t b, uint64_t c) : space(b, c) {}
};

nvshmemi_amd_mspace_t *nvshmemi_amd_mspace_create(uint64_t base, uint64_t capacity) {
    return new nvshmemi_amd_mspace(base, capacity);
}
void nvshmemi_amd_mspace_destroy(nvshmemi_amd_mspace_t *m) { delete m; }
uint64_t nvshmemi_amd_mspace_allocate(nvshmemi_amd_mspace_t *m, uint64_t bytes) {
    return m->space.allocate(bytes);
}
uint64_t nvshmemi_amd_mspace_allocate_aligned(nvshmemi_amd_mspace_t *m, uint64_t alignment,
                                              uint64_t bytes) {
    return m->space.allocate_aligned(alignment, bytes);
}
int nvshmemi_amd_mspace_deallocate(nvshmemi_amd_mspace_t *m, uint64_t addr) {
    return m->space.deallocate(addr) ? 0 : -1;
}
uint64_t nvshmemi_amd_mspace_reallocate(nvshmemi_amd_mspace_t *m, uint64_t addr, uint64_t bytes,
                                        uint64_t *moved_from) {
    return m->space.reallocate(addr, bytes, moved_from);
}
uint64_t nvshmemi_amd_mspace_inuse_size(nvshmemi_amd_mspace_t *m, uint64_t addr) {
    return m->space.inuse_size(addr);
}
uint64_t nvshmemi_amd_mspace_free_bytes(nvshmemi_amd_mspace_t *m) { return m->space.free_bytes(); }
uint64_t nvshmemi_amd_mspace_free_chunks(nvshmemi_amd_mspace_t *m) { return m->space.free_chunks(); }

}  // extern "C"
