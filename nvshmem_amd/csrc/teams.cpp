// Teams of logical PEs (reference src/host/team/team.cu:19-115, team_internal.cpp:2182-2349).
//
// The reference keeps, on every PE, one nvshmemi_team_t per handle describing the team that PE
// belongs to.  Here the host thread stands for all PEs, so the table holds that description for
// every (handle, PE) pair, and one handle can name a family of disjoint teams (all rows of a 2-D
// split).  No per-team scratch is carved from the heap: the only per-team state the load/store
// collectives need is one row of barrier arrival words per PE.
#include <cstdlib>
#include <cstring>

#include "nvshmem.h"
#include "runtime.hpp"

namespace nvshmem_amd {
namespace {

constexpr int kMaxTeams = NVSHMEMI_AMD_MAX_TEAMS;
constexpr int kMaxPes = NVSHMEMI_AMD_MAX_PES;

const nvshmemi_amd_team_view_t kNotMember = {0, 1, 0, -1};

bool handle_ok(const Runtime &rt, nvshmem_team_t team) {
    return team >= 0 && team < kMaxTeams && rt.teams.used[team];
}

size_t ll_bytes_per_team(const Runtime &rt) {
    return (size_t)rt.npes * NVSHMEMI_AMD_LL_BUFFERS * 2 * NVSHMEMI_AMD_LL_PAYLOAD_BYTES;
}

// the staging buffers of all teams follow the packet buffers of all teams in one allocation
size_t stage_bytes_per_team(const Runtime &rt) {
    return (size_t)rt.npes * NVSHMEMI_AMD_STAGE_BUFFERS * NVSHMEMI_AMD_STAGE_BYTES;
}

// distinct member sets of the handle, in order of their first PE
void rebuild_groups(Runtime &rt, int team) {
    TeamTable &tt = rt.teams;
    int n = 0;
    for (int pe = 0; pe < rt.npes; ++pe) {
        const nvshmemi_amd_team_view_t &v = tt.views[team][pe];
        if (v.size <= 0 || v.my_pe != 0) continue;  // each team is listed by its first member
        tt.groups[team][n] = v;
        tt.groups[team][n].my_pe = 0;
        ++n;
    }
    tt.ngroups[team] = n;
}

bool upload_team(Runtime &rt, int team) {
    TeamTable &tt = rt.teams;
    rebuild_groups(rt, team);
    const size_t row = sizeof(nvshmemi_amd_team_view_t) * kMaxPes;
    hipError_t e = hipMemcpy(tt.dev_views() + (size_t)team * kMaxPes, tt.views[team], row,
                             hipMemcpyHostToDevice);
    if (e == hipSuccess)
        e = hipMemcpy(tt.dev_groups() + (size_t)team * kMaxPes, tt.groups[team], row,
                      hipMemcpyHostToDevice);
    // a reused handle must not see the epochs of its previous members
    if (e == hipSuccess)
        e = hipMemset(tt.dev_sync() + (size_t)team * kMaxPes * NVSHMEMI_AMD_TEAM_SYNC_WORDS, 0,
                      sizeof(uint64_t) * kMaxPes * NVSHMEMI_AMD_TEAM_SYNC_WORDS);
    // ... nor packets whose flags its restarted call counter would accept
    if (e == hipSuccess && tt.ll)
        e = hipMemset(tt.ll + (size_t)team * ll_bytes_per_team(rt), 0, ll_bytes_per_team(rt));
    if (e != hipSuccess) {
        set_error("team table upload failed: %s", hipGetErrorString(e));
        return false;
    }
    return true;
}

void set_all(Runtime &rt, int team, int start, int stride, int size) {
    for (int pe = 0; pe < kMaxPes; ++pe) rt.teams.views[team][pe] = kNotMember;
    for (int i = 0; i < size; ++i) rt.teams.views[team][start + i * stride] = {start, stride, size, i};
    rt.teams.used[team] = true;
}

void default_config(nvshmem_team_config_t *c) {
    memset(c, 0, sizeof *c);
    c->version = NVSHMEMI_TEAM_CONFIG_VERSION_2_IDENTIFIER;
    c->num_contexts = -1;
    c->uniqueid = (nvshmemx_team_uniqueid_t)-1;
}

int free_handle(const Runtime &rt) {
    for (int t = NVSHMEM_TEAMS_MIN; t < kMaxTeams; ++t)
        if (!rt.teams.used[t]) return t;
    return NVSHMEM_TEAM_INVALID;
}

bool require(Runtime &rt, const char *what) {
    if (!rt.initialized) {
        set_error("%s called before nvshmem_init", what);
        return false;
    }
    return true;
}

// Child triple of one parent team (team_internal.cpp:2197-2222).  False: arguments rejected.
bool child_of(const Runtime &rt, const nvshmemi_amd_team_view_t &parent, int start, int stride,
              int size, nvshmemi_amd_team_view_t *child) {
    if (start < 0 || start >= parent.size || size <= 0 || size > parent.size || stride < 1)
        return false;
    const int g_start = parent.start + start * parent.stride;
    const int g_stride = parent.stride * stride;
    const int g_end = g_start + g_stride * (size - 1);
    if (g_start >= rt.npes || g_end >= rt.npes) return false;
    *child = {g_start, g_stride, size, 0};
    return true;
}

void record_config(Runtime &rt, int team, const nvshmem_team_config_t *config, long mask) {
    if (config) {
        rt.teams.config[team] = *config;
        rt.teams.config_mask[team] = mask;
    } else {
        default_config(&rt.teams.config[team]);
        rt.teams.config_mask[team] = 0;
    }
}

}  // namespace

bool teams_init(Runtime &rt) {
    TeamTable &tt = rt.teams;
    const size_t views_bytes = sizeof(nvshmemi_amd_team_view_t) * kMaxTeams * kMaxPes;
    const size_t sync_bytes = sizeof(uint64_t) * kMaxTeams * kMaxPes * NVSHMEMI_AMD_TEAM_SYNC_WORDS;
    void *mem = nullptr;
    hipError_t e = hipMalloc(&mem, 2 * views_bytes + sync_bytes);
    if (e != hipSuccess || !mem) {
        (void)hipGetLastError();
        set_error("team table: hipMalloc of %zu bytes failed: %s", 2 * views_bytes + sync_bytes,
                  hipGetErrorString(e));
        return false;
    }
    tt.dev = (char *)mem;
    if (hipMemset(mem, 0, 2 * views_bytes + sync_bytes) != hipSuccess) {
        set_error("team table: hipMemset failed");
        return false;
    }
    // packet buffers of the low-latency collectives; NVSHMEM_AMD_DISABLE_LL=1 leaves them out and
    // every in-kernel collective takes its copy-and-barrier path
    const char *no_ll = getenv("NVSHMEM_AMD_DISABLE_LL");
    if (!(no_ll && no_ll[0] == '1')) {
        const size_t ll_bytes = (ll_bytes_per_team(rt) + stage_bytes_per_team(rt)) * kMaxTeams;
        e = hipMalloc(&mem, ll_bytes);
        if (e != hipSuccess || !mem) {
            (void)hipGetLastError();
            set_error("team table: hipMalloc of %zu bytes of packet buffers failed: %s", ll_bytes,
                      hipGetErrorString(e));
            return false;
        }
        tt.ll = (char *)mem;
        if (hipMemset(mem, 0, ll_bytes) != hipSuccess) {
            set_error("team table: hipMemset failed");
            return false;
        }
    }
    for (int t = 0; t < kMaxTeams; ++t) {
        tt.used[t] = false;
        tt.ngroups[t] = 0;
        tt.config_mask[t] = 0;
        default_config(&tt.config[t]);
        for (int pe = 0; pe < kMaxPes; ++pe) tt.views[t][pe] = kNotMember;
    }
    // every logical PE shares the one GPU: SHARED, NODE and SAME_GPU are the whole world,
    // SAME_MYPE_NODE is each PE alone, GPU_LEADERS is PE 0 (team_internal.cpp:942-1240)
    set_all(rt, NVSHMEM_TEAM_WORLD, 0, 1, rt.npes);
    set_all(rt, NVSHMEM_TEAM_SHARED, 0, 1, rt.npes);
    set_all(rt, NVSHMEMX_TEAM_NODE, 0, 1, rt.npes);
    set_all(rt, NVSHMEMI_TEAM_SAME_GPU, 0, 1, rt.npes);
    set_all(rt, NVSHMEMI_TEAM_GPU_LEADERS, 0, 1, 1);
    for (int pe = 0; pe < kMaxPes; ++pe)
        tt.views[NVSHMEMX_TEAM_SAME_MYPE_NODE][pe] = pe < rt.npes ? nvshmemi_amd_team_view_t{pe, 1, 1, 0} : kNotMember;
    tt.used[NVSHMEMX_TEAM_SAME_MYPE_NODE] = true;
    for (int t = 0; t < NVSHMEM_TEAMS_MIN; ++t)
        if (!upload_team(rt, t)) return false;
    rt.dev.team_views = tt.dev_views();
    rt.dev.team_sync = tt.dev_sync();
    rt.dev.ll_buffers = tt.ll;
    return true;
}

void teams_finalize(Runtime &rt) {
    if (rt.teams.dev) (void)hipFree(rt.teams.dev);
    if (rt.teams.ll) (void)hipFree(rt.teams.ll);
    rt.teams.dev = nullptr;
    rt.teams.ll = nullptr;
    for (int t = 0; t < kMaxTeams; ++t) rt.teams.used[t] = false;
}

bool resolve_team(Runtime &rt, const char *what, nvshmem_team_t team, TeamLaunch *out) {
    if (!require(rt, what)) return false;
    if (!handle_ok(rt, team)) {
        set_error("%s: team %d does not exist", what, (int)team);
        return false;
    }
    const TeamTable &tt = rt.teams;
    out->groups = tt.dev_groups() + (size_t)team * kMaxPes;
    out->ngroups = tt.ngroups[team];
    out->max_size = 0;
    out->min_size = kMaxPes + 1;
    for (int g = 0; g < out->ngroups; ++g) {
        const int n = tt.groups[team][g].size;
        if (n > out->max_size) out->max_size = n;
        if (n < out->min_size) out->min_size = n;
    }
    if (out->ngroups == 0) {
        set_error("%s: team %d has no members", what, (int)team);
        return false;
    }
    return true;
}

}  // namespace nvshmem_amd

using namespace nvshmem_amd;

extern "C" {

int nvshmem_team_my_pe(nvshmem_team_t team) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!rt.initialized || !handle_ok(rt, team)) return -1;
    const nvshmemi_amd_team_view_t &v = rt.teams.views[team][0];
    return v.size > 0 ? v.my_pe : -1;
}

int nvshmem_team_n_pes(nvshmem_team_t team) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!rt.initialized || !handle_ok(rt, team)) return -1;
    const nvshmemi_amd_team_view_t &v = rt.teams.views[team][0];
    return v.size > 0 ? v.size : -1;
}

void nvshmem_team_get_config(nvshmem_team_t team, nvshmem_team_config_t *config) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!config || !rt.initialized || !handle_ok(rt, team)) return;
    *config = rt.teams.config[team];
}

int nvshmem_team_translate_pe(nvshmem_team_t src_team, int src_pe, nvshmem_team_t dest_team) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!rt.initialized || !handle_ok(rt, src_team) || !handle_ok(rt, dest_team)) return -1;
    const nvshmemi_amd_team_view_t &s = rt.teams.views[src_team][0];
    const nvshmemi_amd_team_view_t &d = rt.teams.views[dest_team][0];
    // team_internal.cpp:579-589: an index equal to the size wraps to member 0, larger ones fail
    if (s.size <= 0 || d.size <= 0 || src_pe < 0 || src_pe > s.size) return -1;
    const int off = s.start + (src_pe % s.size) * s.stride - d.start;
    if (off < 0 || off % d.stride != 0 || off / d.stride >= d.size) return -1;
    return off / d.stride;
}

int nvshmemx_amd_team_view(nvshmem_team_t team, int pe, int view[4]) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (!require(rt, "nvshmemx_amd_team_view")) return NVSHMEMX_ERROR_INVALID_VALUE;
    if (!handle_ok(rt, team) || pe < 0 || pe >= rt.npes || !view) {
        set_error("nvshmemx_amd_team_view: team %d / pe %d does not exist", (int)team, pe);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    const nvshmemi_amd_team_view_t &v = rt.teams.views[team][pe];
    view[0] = v.start;
    view[1] = v.stride;
    view[2] = v.size;
    view[3] = v.my_pe;
    return 0;
}

int nvshmem_team_split_strided(nvshmem_team_t parent_team, int PE_start, int PE_stride,
                               int PE_size, const nvshmem_team_config_t *config, long config_mask,
                               nvshmem_team_t *new_team) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (new_team) *new_team = NVSHMEM_TEAM_INVALID;
    if (!require(rt, "nvshmem_team_split_strided") || !new_team) return NVSHMEMX_ERROR_INVALID_VALUE;
    if (parent_team == NVSHMEM_TEAM_INVALID) return NVSHMEMX_ERROR_INVALID_VALUE;  // team.cu:65-68
    if (!handle_ok(rt, parent_team)) {
        set_error("nvshmem_team_split_strided: parent team %d does not exist", (int)parent_team);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    TeamTable &tt = rt.teams;
    nvshmemi_amd_team_view_t fresh[kMaxPes];
    for (int pe = 0; pe < kMaxPes; ++pe) fresh[pe] = kNotMember;
    for (int g = 0; g < tt.ngroups[parent_team]; ++g) {
        const nvshmemi_amd_team_view_t &parent = tt.groups[parent_team][g];
        nvshmemi_amd_team_view_t child;
        if (!child_of(rt, parent, PE_start, PE_stride, PE_size, &child)) {
            set_error("nvshmem_team_split_strided: invalid <start, stride, size>: child <%d, %d, %d>, "
                      "parent <%d, %d, %d>", PE_start, PE_stride, PE_size, parent.start,
                      parent.stride, parent.size);
            return NVSHMEMX_ERROR_INVALID_VALUE;
        }
        for (int i = 0; i < child.size; ++i) {
            child.my_pe = i;
            fresh[child.start + i * child.stride] = child;
        }
    }
    const int t = free_handle(rt);
    if (t == NVSHMEM_TEAM_INVALID) {
        set_error("nvshmem_team_split_strided: all %d team handles are in use", kMaxTeams);
        return NVSHMEMX_ERROR_OUT_OF_MEMORY;
    }
    // the reference synchronises the parent around the split (team_internal.cpp:2228, :2267-2268)
    NVSHMEM_AMD_HIP_CHECK(hipDeviceSynchronize());
    memcpy(tt.views[t], fresh, sizeof fresh);
    tt.used[t] = true;
    record_config(rt, t, config, config_mask);
    if (!upload_team(rt, t)) {
        tt.used[t] = false;
        return NVSHMEMX_ERROR_INTERNAL;
    }
    *new_team = t;
    return 0;
}

int nvshmem_team_split_2d(nvshmem_team_t parent_team, int xrange,
                          const nvshmem_team_config_t *xaxis_config, long xaxis_mask,
                          nvshmem_team_t *xaxis_team, const nvshmem_team_config_t *yaxis_config,
                          long yaxis_mask, nvshmem_team_t *yaxis_team) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (xaxis_team) *xaxis_team = NVSHMEM_TEAM_INVALID;
    if (yaxis_team) *yaxis_team = NVSHMEM_TEAM_INVALID;
    if (!require(rt, "nvshmem_team_split_2d") || !xaxis_team || !yaxis_team)
        return NVSHMEMX_ERROR_INVALID_VALUE;
    if (parent_team == NVSHMEM_TEAM_INVALID) return NVSHMEMX_ERROR_INVALID_VALUE;  // team.cu:92-96
    if (!handle_ok(rt, parent_team) || xrange < 1) {
        set_error("nvshmem_team_split_2d: parent team %d / xrange %d invalid", (int)parent_team, xrange);
        return NVSHMEMX_ERROR_INVALID_VALUE;
    }
    TeamTable &tt = rt.teams;
    const int tx = free_handle(rt);
    if (tx != NVSHMEM_TEAM_INVALID) tt.used[tx] = true;  // reserve while looking for the second
    const int ty = free_handle(rt);
    if (tx != NVSHMEM_TEAM_INVALID) tt.used[tx] = false;
    if (tx == NVSHMEM_TEAM_INVALID || ty == NVSHMEM_TEAM_INVALID) {
        set_error("nvshmem_team_split_2d: fewer than two of the %d team handles are free", kMaxTeams);
        return NVSHMEMX_ERROR_OUT_OF_MEMORY;
    }
    for (int pe = 0; pe < kMaxPes; ++pe) tt.views[tx][pe] = tt.views[ty][pe] = kNotMember;
    // team_internal.cpp:2292-2349: rows are runs of xrange consecutive members (the last may be
    // shorter), columns take every xrange-th member (the first `remainder` columns are one longer)
    for (int g = 0; g < tt.ngroups[parent_team]; ++g) {
        const nvshmemi_amd_team_view_t &parent = tt.groups[parent_team][g];
        const int n = parent.size;
        const int xr = xrange > n ? n : xrange;
        const int rows = (n + xr - 1) / xr, rem = n % xr;
        for (int i = 0; i < n; ++i) {
            const int pe = parent.start + i * parent.stride;
            const int row = i / xr, col = i % xr;
            const int xsize = (row == rows - 1 && rem) ? rem : xr;
            const int ysize = (rem && col < rem) ? n / xr + 1 : n / xr;
            tt.views[tx][pe] = {parent.start + row * xr * parent.stride, parent.stride, xsize, col};
            tt.views[ty][pe] = {parent.start + col * parent.stride, parent.stride * xr, ysize, row};
        }
    }
    NVSHMEM_AMD_HIP_CHECK(hipDeviceSynchronize());
    tt.used[tx] = tt.used[ty] = true;
    record_config(rt, tx, xaxis_config, xaxis_mask);
    record_config(rt, ty, yaxis_config, yaxis_mask);
    if (!upload_team(rt, tx) || !upload_team(rt, ty)) {
        tt.used[tx] = tt.used[ty] = false;
        return NVSHMEMX_ERROR_INTERNAL;
    }
    *xaxis_team = tx;
    *yaxis_team = ty;
    return 0;
}

void nvshmem_team_destroy(nvshmem_team_t team) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    if (team == NVSHMEM_TEAM_INVALID || !rt.initialized) return;
    if (team >= 0 && team < NVSHMEM_TEAMS_MIN) {
        set_error("nvshmem_team_destroy: cannot destroy a pre-defined team (%d)", (int)team);
        return;
    }
    if (!handle_ok(rt, team)) {
        set_error("nvshmem_team_destroy: team %d does not exist", (int)team);
        return;
    }
    // kernels that still use the handle finish first
    NVSHMEM_AMD_HIP_CHECK(hipDeviceSynchronize());
    for (int pe = 0; pe < kMaxPes; ++pe) rt.teams.views[team][pe] = kNotMember;
    (void)upload_team(rt, team);
    rt.teams.used[team] = false;
    rt.teams.ngroups[team] = 0;
}

}  // extern "C"
