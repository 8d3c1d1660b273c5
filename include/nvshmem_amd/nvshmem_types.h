/*
 * Type lists and the device state block.
 *
 * The X-macro lists restate the type matrices of the reference API
 * (reference src/include/device_host/nvshmem_common.cuh:48-73 RMA types, :135-147 sizes,
 * :156-170 wait types, :172-210 reduce types).  Each entry is X(api_name, c_type, kernel_tag):
 * kernel_tag names the one kernel instantiation several same-width C types share
 * (i8..i64, u8..u64, f16, bf16, f32, f64), so `long`, `long long` and `int64_t` run the same code.
 */
#ifndef NVSHMEM_AMD_TYPES_H
#define NVSHMEM_AMD_TYPES_H

#include "nvshmem_constants.h"

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
typedef __hip_bfloat16 nvshmem_bfloat16_t;
typedef __half nvshmem_half_t;
#else
/* Storage-only views for C and host C++ callers: the ABI passes pointers to 2-byte elements. */
typedef struct { uint16_t bits; } nvshmem_bfloat16_t;
typedef struct { uint16_t bits; } nvshmem_half_t;
#endif

/* 25 standard RMA types. */
#define NVSHMEMI_REPT_FOR_STANDARD_RMA_TYPES(X) \
    X(bfloat16, nvshmem_bfloat16_t, bf16)       \
    X(half, nvshmem_half_t, f16)                \
    X(float, float, f32)                        \
    X(double, double, f64)                      \
    X(char, char, i8)                           \
    X(short, short, i16)                        \
    X(schar, signed char, i8)                   \
    X(int, int, i32)                            \
    X(long, long, i64)                          \
    X(longlong, long long, i64)                 \
    X(uchar, unsigned char, u8)                 \
    X(ushort, unsigned short, u16)              \
    X(uint, unsigned int, u32)                  \
    X(ulong, unsigned long, u64)                \
    X(ulonglong, unsigned long long, u64)       \
    X(int8, int8_t, i8)                         \
    X(int16, int16_t, i16)                      \
    X(int32, int32_t, i32)                      \
    X(int64, int64_t, i64)                      \
    X(uint8, uint8_t, u8)                       \
    X(uint16, uint16_t, u16)                    \
    X(uint32, uint32_t, u32)                    \
    X(uint64, uint64_t, u64)                    \
    X(size, size_t, u64)                        \
    X(ptrdiff, ptrdiff_t, i64)

/* put8/16/32/64/128: element width in bits and bytes. */
#define NVSHMEMI_REPT_FOR_SIZES(X) X(8, 1) X(16, 2) X(32, 4) X(64, 8) X(128, 16)

/* 14 wait/test types. */
#define NVSHMEMI_REPT_FOR_WAIT_TYPES(X) \
    X(short, short)                     \
    X(int, int)                         \
    X(long, long)                       \
    X(longlong, long long)              \
    X(ushort, unsigned short)           \
    X(uint, unsigned int)               \
    X(ulong, unsigned long)             \
    X(ulonglong, unsigned long long)    \
    X(int32, int32_t)                   \
    X(int64, int64_t)                   \
    X(uint32, uint32_t)                 \
    X(uint64, uint64_t)                 \
    X(size, size_t)                     \
    X(ptrdiff, ptrdiff_t)

/* Atomic memory operations (reference src/include/host/nvshmem_api.h:91-112): fetch / set / swap /
 * compare_swap / inc / add exist for the bitwise and the standard lists, fetch / set / swap also
 * for the extended list, and / or / xor for the bitwise list only. */
#define NVSHMEMI_REPT_FOR_BITWISE_AMO_TYPES(X) \
    X(uint, unsigned int)                      \
    X(ulong, unsigned long)                    \
    X(ulonglong, unsigned long long)           \
    X(int32, int32_t)                          \
    X(int64, int64_t)                          \
    X(uint32, uint32_t)                        \
    X(uint64, uint64_t)
#define NVSHMEMI_REPT_FOR_STANDARD_AMO_TYPES(X) \
    NVSHMEMI_REPT_FOR_BITWISE_AMO_TYPES(X)      \
    X(int, int)                                 \
    X(long, long)                               \
    X(longlong, long long)                      \
    X(size, size_t)                             \
    X(ptrdiff, ptrdiff_t)
#define NVSHMEMI_REPT_FOR_EXTENDED_AMO_TYPES(X) \
    X(float, float)                             \
    X(double, double)

/* Operation ids of the reference's nvshmemi_amo_t
 * (src/include/device_host_transport/nvshmem_common_transport.h:41-62). */
typedef enum {
    NVSHMEMI_AMO_INC = 2,
    NVSHMEMI_AMO_SET = 3,
    NVSHMEMI_AMO_ADD = 4,
    NVSHMEMI_AMO_AND = 5,
    NVSHMEMI_AMO_OR = 6,
    NVSHMEMI_AMO_XOR = 7,
    NVSHMEMI_AMO_FETCH = 12,
    NVSHMEMI_AMO_FETCH_INC = 13,
    NVSHMEMI_AMO_FETCH_ADD = 14,
    NVSHMEMI_AMO_FETCH_AND = 15,
    NVSHMEMI_AMO_FETCH_OR = 16,
    NVSHMEMI_AMO_FETCH_XOR = 17,
    NVSHMEMI_AMO_SWAP = 18,
    NVSHMEMI_AMO_COMPARE_SWAP = 19
} nvshmemi_amo_t;

/* and / or / xor. */
#define NVSHMEMI_REPT_FOR_BITWISE_REDUCE_TYPES(X, OP) \
    X(uchar, unsigned char, u8, OP)                   \
    X(ushort, unsigned short, u16, OP)                \
    X(uint, unsigned int, u32, OP)                    \
    X(ulong, unsigned long, u64, OP)                  \
    X(ulonglong, unsigned long long, u64, OP)         \
    X(int8, int8_t, i8, OP)                           \
    X(int16, int16_t, i16, OP)                        \
    X(int32, int32_t, i32, OP)                        \
    X(int64, int64_t, i64, OP)                        \
    X(uint8, uint8_t, u8, OP)                         \
    X(uint16, uint16_t, u16, OP)                      \
    X(uint32, uint32_t, u32, OP)                      \
    X(uint64, uint64_t, u64, OP)                      \
    X(size, size_t, u64, OP)

/* min / max / sum / prod: the bitwise list plus the signed and floating types. */
#define NVSHMEMI_REPT_FOR_STANDARD_REDUCE_TYPES(X, OP) \
    NVSHMEMI_REPT_FOR_BITWISE_REDUCE_TYPES(X, OP)      \
    X(char, char, i8, OP)                              \
    X(schar, signed char, i8, OP)                      \
    X(short, short, i16, OP)                           \
    X(int, int, i32, OP)                               \
    X(long, long, i64, OP)                             \
    X(longlong, long long, i64, OP)                    \
    X(bfloat16, nvshmem_bfloat16_t, bf16, OP)          \
    X(half, nvshmem_half_t, f16, OP)                   \
    X(float, float, f32, OP)                           \
    X(double, double, f64, OP)

/* Every (type, op) pair of the reduce API, in one list: X(api_name, c_type, kernel_tag, op). */
#define NVSHMEMI_REPT_FOR_ALL_REDUCE_TYPES_AND_OPS(X) \
    NVSHMEMI_REPT_FOR_BITWISE_REDUCE_TYPES(X, and)    \
    NVSHMEMI_REPT_FOR_BITWISE_REDUCE_TYPES(X, or)     \
    NVSHMEMI_REPT_FOR_BITWISE_REDUCE_TYPES(X, xor)    \
    NVSHMEMI_REPT_FOR_STANDARD_REDUCE_TYPES(X, max)   \
    NVSHMEMI_REPT_FOR_STANDARD_REDUCE_TYPES(X, min)   \
    NVSHMEMI_REPT_FOR_STANDARD_REDUCE_TYPES(X, sum)   \
    NVSHMEMI_REPT_FOR_STANDARD_REDUCE_TYPES(X, prod)

/* Reduction operator ids shared by host launchers, device code and the test oracle
 * (same set as the reference's rdxn_ops_t, src/include/device_host/nvshmem_common.cuh:471-489). */
typedef enum {
    NVSHMEMI_OP_and = 0,
    NVSHMEMI_OP_or = 1,
    NVSHMEMI_OP_xor = 2,
    NVSHMEMI_OP_min = 3,
    NVSHMEMI_OP_max = 4,
    NVSHMEMI_OP_sum = 5,
    NVSHMEMI_OP_prod = 6
} nvshmemi_amd_op_t;

/* Element kinds of the shared kernel instantiations. */
typedef enum {
    NVSHMEMI_DT_i8 = 0,
    NVSHMEMI_DT_i16,
    NVSHMEMI_DT_i32,
    NVSHMEMI_DT_i64,
    NVSHMEMI_DT_u8,
    NVSHMEMI_DT_u16,
    NVSHMEMI_DT_u32,
    NVSHMEMI_DT_u64,
    NVSHMEMI_DT_f16,
    NVSHMEMI_DT_bf16,
    NVSHMEMI_DT_f32,
    NVSHMEMI_DT_f64,
    NVSHMEMI_DT_COUNT
} nvshmemi_amd_dtype_t;

/*
 * State block read by device code (counterpart of the reference's nvshmemi_device_host_state_t,
 * src/include/device_host/nvshmem_types.h:452-509).  All logical PEs live in one allocation:
 * PE p owns [heap_base + p*heap_size, heap_base + (p+1)*heap_size), heap_size being the distance
 * between slices (a multiple of 2 MiB, of 16 MiB for large heaps; no power of two), so the
 * reference's peer_heap_base_p2p[] table collapses to a multiplication.  Symmetric addresses handed
 * to users are addresses inside PE 0's slice ("canonical" addresses).
 */
/* Team `t` as PE `p` sees it: entry [t * NVSHMEMI_AMD_MAX_PES + p] of the team table.  The
 * members are the world PEs start + i*stride, i < size; my_pe is p's index among them.  size == 0:
 * p is not a member (its handle would be NVSHMEM_TEAM_INVALID in the reference).  One handle can
 * thus name a family of disjoint teams, e.g. every row of a 2-D split, and a collective called
 * once serves all of them.  Counterpart of the start/stride/size/my_pe fields of nvshmemi_team_t
 * (src/include/device_host/nvshmem_types.h:312-343). */
typedef struct {
    int32_t start, stride, size, my_pe;
} nvshmemi_amd_team_view_t;

/* Arrival words of a team barrier: NVSHMEMI_AMD_MAX_PES words indexed by the sender's member
 * index, then the PE's epoch; one such row per (team, PE). */
#define NVSHMEMI_AMD_TEAM_SYNC_WORDS (NVSHMEMI_AMD_MAX_PES + 8)

/* Low-latency collectives: every (team, PE) owns NVSHMEMI_AMD_LL_BUFFERS packet buffers (used in
 * rotation, by the team's call counter) that hold 16-byte packets for NVSHMEMI_AMD_LL_PAYLOAD_BYTES bytes of
 * payload each.  A PE's contribution travels that way when it is at most
 * NVSHMEMI_AMD_LL_MAX_BYTES long and all contributions of the team fit one buffer.  Word
 * NVSHMEMI_AMD_LL_COUNT_WORD of a PE's team sync row counts the team's low-latency calls,
 * NVSHMEMI_AMD_LL_DONE_WORD publishes the last one the PE has finished reading. */
#define NVSHMEMI_AMD_LL_BUFFERS 3
#define NVSHMEMI_AMD_LL_PAYLOAD_BYTES 16384
#define NVSHMEMI_AMD_LL_MAX_BYTES 2048
#define NVSHMEMI_AMD_LL_BCAST_MAX_BYTES 16384 /* broadcast: one contribution, up to a whole buffer */
/* Behind the packet buffers of all teams every (team, PE) owns NVSHMEMI_AMD_STAGE_BUFFERS staging
 * buffers of NVSHMEMI_AMD_STAGE_BYTES: the members of a small in-kernel reduction push their whole
 * contributions there (member i into slot i) and every PE folds its own copy after ONE barrier; the
 * parity of the team's barrier count picks the buffer. */
#define NVSHMEMI_AMD_STAGE_BUFFERS 2
#define NVSHMEMI_AMD_STAGE_BYTES 32768
#define NVSHMEMI_AMD_LL_COUNT_WORD (NVSHMEMI_AMD_MAX_PES + 1)
#define NVSHMEMI_AMD_LL_DONE_WORD (NVSHMEMI_AMD_MAX_PES + 2)
/* Words of a PE's team sync row where the wavefronts of nvshmemx_barrier_warpgroup meet: the
 * arrival count (zero between meetings) and, one word on, the generation. */
#define NVSHMEMI_AMD_WARPGROUP_ARRIVE_WORD (NVSHMEMI_AMD_MAX_PES + 3)
#define NVSHMEMI_AMD_WARPGROUP_SIZE 256 /* four wavefronts, as the reference's warpgroup is four warps */

typedef struct nvshmemi_device_state {
    uint32_t version;     /* (1 << 16) + sizeof(struct) */
    int32_t mype;         /* PE a kernel acts as when its grid is not PE-multiplexed */
    int32_t npes;
    uint32_t options;     /* NVSHMEMI_AMD_OPTION_* bits */
    char *heap_base;      /* start of PE 0's slice */
    uint64_t heap_size;   /* bytes from one PE's slice to the next (a multiple of 2 MiB, of 16 MiB for large heaps) */
    uint64_t *sync_flags; /* canonical address: NVSHMEMI_AMD_MAX_PES arrival words per PE */
    uint64_t *sync_epoch; /* canonical address: that PE's barrier epoch */
    uint64_t spin_limit;  /* 0 = wait forever; else a bounded wait gives up after this many polls */
    uint64_t *timeout_record; /* canonical address: 4 words {number of the timeout (0: none), addr, found, expected} */
    const nvshmemi_amd_team_view_t *team_views; /* [NVSHMEMI_AMD_MAX_TEAMS][NVSHMEMI_AMD_MAX_PES] */
    uint64_t *team_sync; /* [MAX_TEAMS][MAX_PES][NVSHMEMI_AMD_TEAM_SYNC_WORDS]: barrier rows of the teams
                            other than WORLD, low-latency counters of all teams */
    char *ll_buffers;    /* [MAX_TEAMS][npes][NVSHMEMI_AMD_LL_BUFFERS][2 * NVSHMEMI_AMD_LL_PAYLOAD_BYTES], then
                            [MAX_TEAMS][npes][NVSHMEMI_AMD_STAGE_BUFFERS][NVSHMEMI_AMD_STAGE_BYTES] */
    uint64_t *runtime_words; /* one copy for the whole GPU (an address in PE 0's slice, used as it is):
                                word NVSHMEMI_AMD_TIMEOUT_COUNT_WORD counts the bounded waits that gave up */
    uint64_t heap_magic;     /* floor(2^40 / (heap_size >> 21)) + 1: the slice that holds heap offset d is
                                ((d >> 21) * heap_magic) >> 40 (exact while the whole heap is at most 512 GiB) */
    uint64_t *timeout_flag;  /* pinned host memory (or null): a bounded wait that gives up stores its timeout's
                                number here too, so that the host's check after a synchronisation is one load and
                                the count is fetched from the GPU only when something happened */
} nvshmemi_device_state_t;

#define NVSHMEMI_AMD_TIMEOUT_COUNT_WORD 0
/* bytes at the end of every PE's slice that the runtime keeps for itself: barrier arrival row, epoch,
 * timeout record and runtime words, 512 bytes each */
#define NVSHMEMI_AMD_INTERNAL_BYTES (4 * 512)

#endif
