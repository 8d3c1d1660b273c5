// Process-wide state of the logical-PE runtime, shared by the host translation units of
// libnvshmem_amd.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <memory>
#include <mutex>
#include <set>
#include <string>

#include "mspace.hpp"
#include "nvshmem_amd/nvshmem_host_api.h"

namespace nvshmem_amd {

// Host mirror of the team table.  views[t][p] is team t as world PE p sees it; groups[t] lists the
// distinct member sets of the handle (one per disjoint team of the family), which is what the
// collective kernels iterate over.  The device copy is one allocation: views | groups | sync words.
struct TeamTable {
    nvshmemi_amd_team_view_t views[NVSHMEMI_AMD_MAX_TEAMS][NVSHMEMI_AMD_MAX_PES];
    nvshmemi_amd_team_view_t groups[NVSHMEMI_AMD_MAX_TEAMS][NVSHMEMI_AMD_MAX_PES];
    int ngroups[NVSHMEMI_AMD_MAX_TEAMS];
    bool used[NVSHMEMI_AMD_MAX_TEAMS];
    nvshmem_team_config_t config[NVSHMEMI_AMD_MAX_TEAMS];
    long config_mask[NVSHMEMI_AMD_MAX_TEAMS];
    char *dev = nullptr;
    char *ll = nullptr;  // packet buffers of the low-latency collectives, per (team, PE)
    nvshmemi_amd_team_view_t *dev_views() const { return (nvshmemi_amd_team_view_t *)dev; }
    nvshmemi_amd_team_view_t *dev_groups() const {
        return dev_views() + NVSHMEMI_AMD_MAX_TEAMS * NVSHMEMI_AMD_MAX_PES;
    }
    uint64_t *dev_sync() const {
        return (uint64_t *)(dev_groups() + NVSHMEMI_AMD_MAX_TEAMS * NVSHMEMI_AMD_MAX_PES);
    }
};

// What a collective kernel needs to serve every team of a handle.
struct TeamLaunch {
    const nvshmemi_amd_team_view_t *groups = nullptr;  // device array, ngroups entries
    int ngroups = 0;
    int max_size = 0, min_size = 0;
};

struct Runtime {
    std::recursive_mutex mu;
    bool initialized = false;
    int device = 0;
    int npes = 0;
    int num_cus = 0;
    uint64_t heap_size = 0;  // bytes from one PE's slice to the next, a multiple of 2 MiB (16 MiB for large heaps)
    char *base = nullptr;    // start of PE 0's slice
    std::unique_ptr<SymmetricSpace> space;
    nvshmemi_device_state_t dev{};
    TeamTable teams{};
    std::set<nvshmemi_amd_state_updater_t> updaters;  // one per translation unit with a state block
    bool symbols_stale = false;
    bool plain_collective_launch = false;  // NVSHMEM_AMD_PLAIN_COLLECTIVE_LAUNCH=1, read at init
    // Host-launched collectives treat sources of more bytes than this (all PEs together) as too
    // large to stay in the Infinity Cache: NVSHMEM_AMD_CACHEABLE_SOURCE_BYTES, read at init
    uint64_t cacheable_source_bytes = (uint64_t)256 << 20;
    // fcollect and broadcast take the chunked form from this many bytes of sources (all PEs together) on:
    // NVSHMEM_AMD_CHUNKED_COPY_BYTES, read at init
    uint64_t chunked_copy_bytes = (uint64_t)128 << 20;
    // Allreduce on teams of 3 to 64 members takes the LDS-staged kernel when the sources of all PEs
    // together hold at least this many bytes (a quarter of it for teams of 17
    // to 32 members, four times for larger ones): NVSHMEM_AMD_LDS_REDUCE_BYTES, read at init
    uint64_t lds_reduce_bytes = (uint64_t)64 << 20;
    // An allreduce beyond the cache takes two steps - fold into member 0, chunked broadcast - instead of the fused
    // kernel from this team size on (NVSHMEM_AMD_TWO_STEP_REDUCE_MEMBERS, read at init; 0 = never) when the
    // sources of all members together hold at least two_step_reduce_bytes (NVSHMEM_AMD_TWO_STEP_REDUCE_BYTES), and
    // from three times the team size at any size
    unsigned two_step_reduce_members = 16;
    uint64_t two_step_reduce_bytes = (uint64_t)512 << 20;
    uint64_t timeouts_seen = 0;  // bounded waits that gave up, as far as the host has reported them
    // pinned host word the GPU writes a timeout's number to (null if it could not be allocated), and the value
    // the host found there at its last report: equal values mean nothing gave up since
    uint64_t *timeout_flag = nullptr;
    uint64_t timeout_flag_seen = 0;

    static Runtime &get();

    // Offset of a symmetric address inside its PE slice; false when p is outside the heap.
    bool offset_of(const void *p, uint64_t *off) const {
        const uint64_t d = (uint64_t)((const char *)p - base);
        if (!initialized || p == nullptr || (const char *)p < base || d >= (uint64_t)npes * heap_size)
            return false;
        *off = d % heap_size;
        return true;
    }
    char *slice(int pe) const { return base + (uint64_t)pe * heap_size; }
};

// Records a message for nvshmemx_amd_last_error() and prints it to stderr.
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();

// After the device has been synchronised: reports bounded device-side waits that gave up since the last
// check (stderr, nvshmemx_amd_last_error) and returns how many there were.
uint64_t report_timeouts(Runtime &rt, const char *where);

// Pushes the state block to every registered translation unit when it changed.
void refresh_symbols(Runtime &rt, bool force);

// Team table: allocation and the predefined teams at init, release at finalize.
bool teams_init(Runtime &rt);
void teams_finalize(Runtime &rt);
// Resolves a handle for a collective; reports unknown handles through set_error.
bool resolve_team(Runtime &rt, const char *what, nvshmem_team_t team, TeamLaunch *out);

// Common argument check of the collectives and RMA calls: [p, p+bytes) must lie inside one PE
// slice.  Returns the offset through *off.
bool check_symmetric_range(Runtime &rt, const char *what, const void *p, uint64_t bytes,
                           uint64_t *off);

#define NVSHMEM_AMD_HIP_CHECK(expr)                                                        \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess) {                                                            \
            ::nvshmem_amd::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                                     __FILE__, __LINE__);                                  \
        }                                                                                  \
    } while (0)

}  // namespace nvshmem_amd
