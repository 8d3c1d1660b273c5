/*
 * ABI constants of the NVSHMEM data-movement path, MI355X (gfx950) build.
 *
 * Every numeric value here is part of the binary contract of the reference API and is kept
 * identical so that callers compiled against the reference's enums keep working:
 *   comparison ops       reference src/include/device_host_transport/nvshmem_constants.h:48-56
 *   thread levels        reference src/include/device_host_transport/nvshmem_constants.h:58-64
 *   init status          reference src/include/device_host_transport/nvshmem_constants.h:79-86
 *   signal ops (9, 10)   reference src/include/device_host_transport/nvshmem_common_transport.h:39
 *   team ids             reference src/include/device_host/nvshmem_common.cuh:405-421
 *   status codes         reference src/include/non_abi/nvshmemx_error.h:37-47
 *   spec version 1.3     reference src/include/device_host_transport/nvshmem_constants.h:29-31
 */
#ifndef NVSHMEM_AMD_CONSTANTS_H
#define NVSHMEM_AMD_CONSTANTS_H

#include <limits.h>
#include <stddef.h>
#include <stdint.h>

#define NVSHMEM_MAJOR_VERSION 1
#define NVSHMEM_MINOR_VERSION 3
#define NVSHMEM_VENDOR_MAJOR_VERSION 3
#define NVSHMEM_VENDOR_MINOR_VERSION 5
#define NVSHMEM_VENDOR_PATCH_VERSION 1
#define NVSHMEM_VENDOR_STRING "NVSHMEM v3.5.1 (MI355X logical-PE build)"
#define NVSHMEM_MAX_NAME_LEN 256

typedef enum {
    NVSHMEM_CMP_EQ = 0,
    NVSHMEM_CMP_NE = 1,
    NVSHMEM_CMP_GT = 2,
    NVSHMEM_CMP_LE = 3,
    NVSHMEM_CMP_LT = 4,
    NVSHMEM_CMP_GE = 5,
    NVSHMEM_CMP_SENTINEL = INT_MAX
} nvshmemx_cmp_type_t;

typedef enum {
    NVSHMEM_THREAD_SINGLE = 0,
    NVSHMEM_THREAD_FUNNELED = 1,
    NVSHMEM_THREAD_SERIALIZED = 2,
    NVSHMEM_THREAD_MULTIPLE = 3
} nvshmemx_thread_support_t;

typedef enum {
    NVSHMEM_STATUS_NOT_INITIALIZED = 0,
    NVSHMEM_STATUS_IS_BOOTSTRAPPED = 1,
    NVSHMEM_STATUS_IS_INITIALIZED = 2,
    NVSHMEM_STATUS_LIMITED_MPG = 3,
    NVSHMEM_STATUS_FULL_MPG = 4
} nvshmemx_init_status_t;

/* Signal operators: the values are those of the reference's AMO enumeration. */
#define NVSHMEM_SIGNAL_SET 9
#define NVSHMEM_SIGNAL_ADD 10
/* May be OR-ed into the sig_op of a device-side put-with-signal: the signal is ordered behind the
 * payload of THIS put only, which is what OpenSHMEM promises for the operation.  Without it the
 * signal is also ordered behind everything else the calling thread group wrote before the call, as
 * in the reference (a full fence in front of its signal), which on this GPU costs a write-back of
 * the XCD's L2 per call.  No counterpart in the reference. */
#define NVSHMEMX_AMD_SIGNAL_PAYLOAD_ONLY 0x100
#define NVSHMEMI_AMD_SIGNAL_OP_MASK 0xff
/* nvshmemi_device_state_t::options, bit 0: every device-side put-with-signal takes the payload-only order,
 * as if NVSHMEMX_AMD_SIGNAL_PAYLOAD_ONLY were OR-ed into its sig_op (NVSHMEM_AMD_PUT_SIGNAL_ORDER=payload
 * in the environment at nvshmem_init, or nvshmemx_amd_set_put_signal_order), so that code written for the
 * reference's API can choose it without touching its call sites. */
#define NVSHMEMI_AMD_OPTION_PUT_SIGNAL_PAYLOAD_ONLY 0x1u

typedef int32_t nvshmem_team_t;
#define NVSHMEM_TEAM_INVALID (-1)
#define NVSHMEM_TEAM_WORLD 0
#define NVSHMEM_TEAM_SHARED 1
#define NVSHMEMX_TEAM_NODE 2
/* Predefined teams, numbered as in the reference (src/include/device_host/nvshmem_common.cuh:
 * 406-421).  All logical PEs share one GPU, so SHARED, NODE and SAME_GPU equal WORLD,
 * SAME_MYPE_NODE holds the calling PE alone and GPU_LEADERS holds PE 0 (only PE 0 is a member). */
#define NVSHMEMX_TEAM_SAME_MYPE_NODE 3
#define NVSHMEMI_TEAM_SAME_GPU 4
#define NVSHMEMI_TEAM_GPU_LEADERS 5
#define NVSHMEM_TEAMS_MIN 6
/* Team handles, predefined ones included (reference default of NVSHMEM_MAX_TEAMS: 32). */
#define NVSHMEMI_AMD_MAX_TEAMS 32

/* Team configuration (reference nvshmem_team_config_v2, src/include/device_host/nvshmem_types.h:
 * 93-105, 294-310): recorded and returned by nvshmem_team_get_config; contexts are not used on a
 * load/store path. */
#define NVSHMEM_TEAM_CONFIG_MASK_NUM_CONTEXTS 0x0000000000000001
#define NVSHMEM_TEAM_CONFIG_MASK_UNIQUEID 0x0000000000000002
typedef uint64_t nvshmemx_team_uniqueid_t;
typedef struct {
    int version;
    int num_contexts;
    nvshmemx_team_uniqueid_t uniqueid;
    char padding[48];
} nvshmem_team_config_t;
#define NVSHMEMI_TEAM_CONFIG_VERSION_2_IDENTIFIER ((2 << 16) + (int)sizeof(nvshmem_team_config_t))
#define NVSHMEM_TEAM_CONFIG_INITIALIZER {NVSHMEMI_TEAM_CONFIG_VERSION_2_IDENTIFIER, -1, (nvshmemx_team_uniqueid_t)-1, {0}}

enum nvshmemx_status {
    NVSHMEMX_SUCCESS = 0,
    NVSHMEMX_ERROR_INVALID_VALUE = 1,
    NVSHMEMX_ERROR_OUT_OF_MEMORY = 2,
    NVSHMEMX_ERROR_NOT_SUPPORTED = 3,
    NVSHMEMX_ERROR_SYMMETRY = 4,
    NVSHMEMX_ERROR_GPU_NOT_SELECTED = 5,
    NVSHMEMX_ERROR_COLLECTIVE_LAUNCH_FAILED = 6,
    NVSHMEMX_ERROR_INTERNAL = 7
};

/* Allocation granule of the symmetric heap (reference NVSHMEMI_MALLOC_ALIGNMENT,
 * src/include/internal/host/custom_malloc.h:18-48). */
#define NVSHMEMI_MALLOC_ALIGNMENT ((size_t)512)

/* A CDNA wavefront has 64 lanes; "_warp" scoped calls are collective over one wavefront. */
#define NVSHMEMI_WARP_SIZE 64

/* Upper bound on logical PEs (flag rows of the in-kernel barrier are sized with it). */
#define NVSHMEMI_AMD_MAX_PES 64

#endif
