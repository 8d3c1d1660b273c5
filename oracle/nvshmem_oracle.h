/*
 * CPU oracle of the NVSHMEM data-movement path.  TEST INFRASTRUCTURE ONLY: it is the checker that
 * tests, the smoke run and the benchmark's cpu_baseline leg compare the GPU library against.
 * Nothing in the shipped library links, loads or calls it.
 *
 * Each function restates the operator semantics of the reference in plain C and cites the reference
 * file:line it follows (paths are relative to the reference tree).  The reference ships no CPU
 * implementation of these device paths, so this is a port of the semantics, not of code.
 *
 * Pinning status (what fixes each function independently of this file):
 *   copies / ring put / fcollect / alltoall / moe maps  brute-force index maps on tiny inputs,
 *       involution and replication invariants, the reference's own known answers
 *       (examples/put-block.cu:93-104);
 *   broadcast / reducescatter   brute force, the reference's known answer for broadcast
 *       (examples/ring-bcast.cu:68-72), slices of the pinned reduce for order-free operators, numpy
 *       folds and hand-evaluated NaN cases for the operand order;
 *   atomic operations     exhaustive small-width tables and random words against Python integers;
 *   team arithmetic       PE sets enumerated by brute force from the definitions (members of the
 *       parent by index, rows and columns of the row-major grid), translate against set lookups;
 *   integer reduce        order-free closed forms, numpy, reference known answer dst[i]==i*npes
 *       (examples/ring-reduce.cu:242-248, examples/user-buffer.cu:141-152);
 *   fp32 / fp16 / bf16 reduce   numpy / torch CPU left folds in the element type, order-sensitive
 *       inputs, NaN and signed-zero cases of the min/max operand rule;
 *   comparison and signal operators   exhaustive tables against Python integers;
 *   nvshmem_ptr           closed form;
 *   allocator model       hand-derived address traces of the reference algorithm plus invariants.
 * No function is left "parity unpinned".
 */
#ifndef NVSHMEM_ORACLE_H
#define NVSHMEM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element kinds and operators: same numbering as include/nvshmem_amd/nvshmem_types.h */
enum { ORC_i8, ORC_i16, ORC_i32, ORC_i64, ORC_u8, ORC_u16, ORC_u32, ORC_u64,
       ORC_f16, ORC_bf16, ORC_f32, ORC_f64, ORC_DT_COUNT };
enum { ORC_and, ORC_or, ORC_xor, ORC_min, ORC_max, ORC_sum, ORC_prod };

size_t oracle_dtype_size(int dtype);
void oracle_set_threads(int nthreads); /* worker threads for the large loops (default: all) */
int oracle_get_threads(void);

/* ---- seeded synthetic inputs: counter-based, element i of PE pe depends only on (seed,pe,i) ---- */
uint64_t oracle_splitmix64(uint64_t x);
uint64_t oracle_rand_u64(uint64_t seed, uint64_t pe, uint64_t index);
void oracle_fill_bytes(uint8_t *out, size_t n, uint64_t seed, uint64_t pe);
void oracle_fill_u64(uint64_t *out, size_t n, uint64_t seed, uint64_t pe);
/* uniform integers in [-2^20, 2^20] */
void oracle_fill_i32_pm2p20(int32_t *out, size_t n, uint64_t seed, uint64_t pe);
void oracle_fill_f32_normal(float *out, size_t n, uint64_t seed, uint64_t pe);
void oracle_fill_bf16_normal(uint16_t *out, size_t n, uint64_t seed, uint64_t pe);
void oracle_fill_f16_normal(uint16_t *out, size_t n, uint64_t seed, uint64_t pe);

/* ---- 16-bit float conversions (round to nearest even) ---- */
float oracle_bf16_to_f32(uint16_t v);
uint16_t oracle_f32_to_bf16(float f);
float oracle_f16_to_f32(uint16_t v);
uint16_t oracle_f32_to_f16(float f);

/* ---- point to point ---- */
/* put/get are byte copies into / out of the target PE's copy of the object. */
void oracle_copy(void *dst, const void *src, size_t bytes);
/* every PE p puts its `bytes` bytes to PE (p+1)%npes: dst[(p+1)%npes] = src[p]; arrays are
 * [npes][bytes] */
void oracle_ring_put(uint8_t *dst, const uint8_t *src, int npes, size_t bytes);
/* every PE p gets from PE (p+1)%npes: dst[p] = src[(p+1)%npes] */
void oracle_ring_get(uint8_t *dst, const uint8_t *src, int npes, size_t bytes);
/* signal update: op 9 = set, 10 = add; returns the new value, or old value for an unknown op */
uint64_t oracle_signal_op(uint64_t current, uint64_t signal, int sig_op);
/* comparison used by wait/test: cmp 0..5 = EQ NE GT LE LT GE on unsigned 64-bit */
int oracle_compare_u64(uint64_t found, int cmp, uint64_t expected);
int oracle_compare_i64(int64_t found, int cmp, int64_t expected);
/* nvshmem_ptr on a heap of npes slices of heap_size bytes starting at heap_base; 0 = NULL */
uint64_t oracle_ptr(uint64_t heap_base, uint64_t heap_size, int npes, uint64_t ptr, int pe);

/* ---- collectives: src is [npes][...] contiguous, outputs as noted ---- */
/* dst[k] = fold over p=0..npes-1 of src[p][k]; dst is ONE PE's result ([nelems]); every PE's dest
 * equals it.  Returns 0, or -1 when op is not defined for dtype. */
int oracle_reduce(int dtype, int op, int npes, size_t nelems, const void *src, void *dst);
/* dst[q][p*seg + k] = src[p][k]; dst is [npes][npes*seg_bytes] */
void oracle_fcollect(int npes, size_t seg_bytes, const uint8_t *src, uint8_t *dst);
/* dst[q][p*seg + k] = src[p][q*seg + k]; src and dst are [npes][npes*seg_bytes] */
void oracle_alltoall(int npes, size_t seg_bytes, const uint8_t *src, uint8_t *dst);

/* dst[q][k] = fold over p of src[p][q*nelems + k], order acc = op(x0, x1); acc = op(acc, x_p) for
 * p >= 2 (operands the other way round than in oracle_reduce); src is [npes][npes*nelems], dst is
 * [npes][nelems].  Returns 0, or -1 when op is not defined for dtype. */
int oracle_reducescatter(int dtype, int op, int npes, size_t nelems, const void *src, void *dst);
/* (value, location) maximum: dst[q][k] = fold over p = 0..npes-1 of src[p][k] with
 * acc = (acc.value > x.value) ? acc : x (equal values: the later PE wins; a NaN x replaces acc);
 * src and dst are [npes][nelems][2] doubles */
void oracle_maxloc_reduce(int npes, size_t nelems, const double *src, double *dst);
/* dst[q][k] = src[root][k] for every q including the root; src, dst are [npes][bytes] */
void oracle_broadcast(int npes, size_t bytes, int root, const uint8_t *src, uint8_t *dst);

/* ---- atomic memory operations: op numbering of include/nvshmem_amd/nvshmem_types.h ----
 * One operation on a word of `bits` (32 or 64) bits holding `current`: returns the new contents,
 * *fetched receives what a fetching form returns (the old contents).  Arithmetic wraps modulo
 * 2^bits; compare_swap stores `value` only when current == cond.  Unknown op: word unchanged. */
uint64_t oracle_amo(int op, int bits, uint64_t current, uint64_t value, uint64_t cond,
                    uint64_t *fetched);

/* ---- teams: a team is the PE set {start + i*stride, i < size} of world PEs ---- */
/* child of `parent` = members start, start+stride, ... (size of them) counted in parent indices.
 * Returns 0, or -1 for the argument errors the reference rejects. */
int oracle_team_split_strided(const int parent[3], int npes_world, int start, int stride, int size,
                              int child[3]);
/* index of team `src`'s member src_pe inside team `dst`, or -1 */
int oracle_team_translate_pe(const int src[3], int src_pe, const int dst[3]);
/* the x (row) and y (column) teams of parent member `index` when the parent is laid out row-major
 * with rows of xrange members; the last row / the right-hand columns may be shorter */
void oracle_team_split_2d(const int parent[3], int xrange, int index, int xteam[3], int yteam[3]);

/* ---- allocator model (independent structure: one ordered block list) ---- */
typedef struct oracle_space oracle_space_t;
oracle_space_t *oracle_space_create(uint64_t base, uint64_t capacity);
void oracle_space_destroy(oracle_space_t *s);
uint64_t oracle_space_alloc(oracle_space_t *s, uint64_t bytes);
uint64_t oracle_space_align(oracle_space_t *s, uint64_t alignment, uint64_t bytes);
int oracle_space_free(oracle_space_t *s, uint64_t addr);
uint64_t oracle_space_realloc(oracle_space_t *s, uint64_t addr, uint64_t bytes, uint64_t *moved_from);
uint64_t oracle_space_free_bytes(const oracle_space_t *s);
uint64_t oracle_space_free_chunks(const oracle_space_t *s);

/* ---- MoE token shuffle model ---- */
/* experts[t*topk + k] for PE pe: topk distinct experts per token drawn Zipf(s) over ranks
 * 1..num_experts (expert id = rank-1), duplicates rejected until distinct. */
void oracle_moe_routing(int32_t *experts, int tokens, int topk, int num_experts, double zipf_s,
                        uint64_t seed, uint64_t pe);
/* Dispatch plan for all PEs.  experts is [npes][tokens*topk].  Outputs:
 *   counts[src][e]            rows PE src sends to expert e                       [npes][E]
 *   seg_base[e][src]          first row, in the receive buffer of PE e/(E/npes), of the segment
 *                             holding rows of (expert e, source src); segments are ordered by
 *                             (expert, source PE)                                 [E][npes]
 *   dest_pe / dest_row[src][t*topk+k]  where that copy of token t lands; within a segment rows keep
 *                             (token, k) order                                    [npes][T*K]
 *   recv_rows[pe]             total rows PE pe receives                           [npes]
 */
void oracle_moe_plan(const int32_t *experts, int npes, int tokens, int topk, int num_experts,
                     int64_t *counts, int64_t *seg_base, int32_t *dest_pe, int64_t *dest_row,
                     int64_t *recv_rows);
/* recv[pe] gets its rows: recv_pe[dest_row] = send[src][t] for every (src,t,k) with dest_pe==pe. */
void oracle_moe_dispatch_one(uint8_t *recv_pe, int pe, const uint8_t *send, int npes, int tokens,
                             int topk, size_t row_bytes, const int32_t *dest_pe,
                             const int64_t *dest_row);
/* combine: out[src][(t*topk+k)] = recv[dest_pe][dest_row]; out_src is one PE's [T*K][row_bytes];
 * recv_ptrs[pe] points at PE pe's receive buffer. */
void oracle_moe_combine_one(uint8_t *out_src, int src, const uint8_t *const *recv_ptrs, int tokens,
                            int topk, size_t row_bytes, const int32_t *dest_pe,
                            const int64_t *dest_row);

#ifdef __cplusplus
}
#endif
#endif
