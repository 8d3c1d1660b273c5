/*
 * C ABI of libnvshmem_amd_perftest.so: kernels written against the public device API (nvshmem.h /
 * nvshmemx.h only, a separate code object from the runtime) and the host drivers that start them.
 * They are this build's counterpart of the reference's device-initiated benchmarks and examples,
 * the only in-tree callers of the device API there:
 *   perftest/device/pt-to-pt/shmem_put_bw.cu, shmem_get_bw.cu          -> ring_rma
 *   perftest/device/pt-to-pt/shmem_put_signal_ping_pong_latency.cu     -> put_signal_pingpong
 *   examples/put-block.cu                                              -> ring_rma (its known answer)
 *   examples/ring-reduce.cu                                            -> ring_reduce
 *   perftest/device/coll/{reduction,fcollect,alltoall,barrier}_latency.cu -> device_* entry points
 *   examples/moe_shuffle.cu                                            -> moe_* entry points
 * All pointers are canonical symmetric addresses from nvshmem_malloc unless noted.  Every entry
 * point returns 0 on success or an nvshmemx_status; work is enqueued on `stream` (a hipStream_t
 * passed as void *, NULL = null stream) and is not waited for.
 */
#ifndef NVSHMEM_PERFTEST_H
#define NVSHMEM_PERFTEST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { NVSHMEM_PERFTEST_SCOPE_THREAD = 0, NVSHMEM_PERFTEST_SCOPE_WARP = 1,
       NVSHMEM_PERFTEST_SCOPE_BLOCK = 2 };

/*
 * Every PE p moves `bytes` bytes between its `src` and PE (p+1)%npes: put (is_get = 0) writes the
 * peer's `dest`, get reads the peer's `src` into the local `dest`.  blocks_per_pe blocks of
 * `threads` threads per PE; block b moves the slice [b*bytes/B, (b+1)*bytes/B) (the last block also
 * takes the remainder; with bytes < B only block 0 works), as shmem_put_bw.cu:26-31 does.  With
 * warp scope each wavefront of a block moves an equal part of the block's slice, with thread scope
 * each thread does.  `iters` back-to-back launches.
 */
int nvshmem_perftest_ring_rma(void *dest, const void *src, size_t bytes, int blocks_per_pe,
                              int threads, int scope, int is_get, int iters, void *stream);

/* Counter calibration: PE 0's `src` -> PE 0's `dst`, `bytes` (multiple of 16) with a plain
 * one-vector-per-thread kernel that uses nothing of the NVSHMEM API.  Reads and writes exactly
 * `bytes` each. */
int nvshmem_perftest_plain_copy(void *dst, const void *src, size_t bytes, void *stream);
/* Stream probes for hardware counters (no counterpart in the reference): every block of every PE reads
 * (write == 0) or writes (1: streaming stores, 2: write-through stores) its contiguous slice of the PE's `bytes` at buf, in the access pattern of a long
 * block-scoped copy with the other side removed; the slice is cut to whole rounds of threads x 128 bytes. */
int nvshmem_perftest_stream_probe(void *buf, size_t bytes, int blocks_per_pe, int threads, int write, void *stream);

/* One launch of an empty kernel named profile_marker_kernel: a boundary that a script reading a profiler's
 * kernel trace can recognise (nvshmem_amd/profile_workloads.py brackets every workload with two). */
int nvshmem_perftest_profile_marker(void *stream);

/* PE p writes value_base + p into word [p] of PE (p+1)%npes's `words` with nvshmem_uint64_p, then
 * (after a barrier) reads word [q] of every PE q's `words`... with nvshmem_uint64_g into
 * out[q] of its own `out`.  words and out hold npes uint64 each. */
int nvshmem_perftest_p_g(uint64_t *words, uint64_t *out, uint64_t value_base, void *stream);

/* The PE identity rule of the device API (the reference's nvshmem_my_pe reads the per-process
 * nvshmemi_device_state_d.mype, src/include/device/nvshmem_defines.h:55-57):
 * a launch of grid (1, 1, grid_z) with one thread per block writes nvshmem_my_pe() of block z to out[z]
 * and nvshmem_n_pes() to out[64 + z].  `out` is any device memory of 128 ints.  A grid whose z extent
 * equals the PE count is a PE grid (block z acts as PE z); any other z extent acts as PE 0. */
int nvshmem_perftest_pe_identity(int *out, int grid_z, void *stream);

/* Each of `threads` threads of one block per PE applies nvshmemx_signal_op(sig, value, sig_op,
 * (p+1)%npes) `reps` times. */
int nvshmem_perftest_signal_op(uint64_t *sig, uint64_t value, int sig_op, int threads, int reps,
                               void *stream);

/* One thread per PE waits with nvshmem_signal_wait_until(sig, cmp, cmp_value) and stores the value
 * the wait returned into its own out[0].  Nobody signals: use it with a preset signal word or with
 * a small spin limit (nvshmemx_amd_set_spin_limit) to exercise the bounded wait. */
int nvshmem_perftest_signal_wait(uint64_t *sig, int cmp, uint64_t cmp_value, uint64_t *out,
                                 void *stream);

/* PE 0 and PE 1 bounce a `bytes` payload `iters` times with nvshmemx_putmem_signal_block and
 * nvshmem_signal_wait_until (shmem_put_signal_ping_pong_latency.cu:29-49).  After it `data` on
 * both PEs holds the payload PE 0 started with and sig == iters on both.  npes must be >= 2. */
int nvshmem_perftest_put_signal_pingpong(void *data, uint64_t *sig, size_t bytes, int iters,
                                         int threads, void *stream);

/* Ordering check of put-with-signal.  Even PEs stream `iters` messages of `bytes` (a multiple of 8) to
 * their odd neighbours, `blocks` independent streams per PE, each through a ring of `slots` buffers:
 * the sender fills its staging buffer with words that depend on (message, block, index), sends it with
 * nvshmemx_putmem_signal_nbi_block (256 threads) / _warp (64) / nvshmem_putmem_signal_nbi (1 thread) and
 * sig_op = NVSHMEM_SIGNAL_ADD, optionally OR-ed with NVSHMEMX_AMD_SIGNAL_PAYLOAD_ONLY; the receiver waits
 * for the count with nvshmem_signal_wait_until(GE), reads the slot at once, adds the number of wrong
 * words to its errors[0] and returns a credit with nvshmemx_signal_op.  data holds blocks * slots *
 * bytes, stage blocks * bytes, sig 2 words per block (zero before the call), errors one word (zero). */
int nvshmem_perftest_put_signal_stream(void *data, void *stage, uint64_t *sig, uint64_t *errors,
                                       size_t bytes, int slots, int iters, int blocks, int scope,
                                       int sig_op, void *stream);

/* Sets nwords 64-bit words of every PE's copy of `words` to `value` with one kernel on `stream` (for
 * clearing signal words between timed launches without a host synchronisation per PE). */
int nvshmem_perftest_fill_words(uint64_t *words, uint64_t value, size_t nwords, void *stream);

/* Latency loops of the reference's perftest/device/pt-to-pt programs, one block per PE, `iters`
 * repetitions inside one launch.  Kinds 0-4: PE 0 acts on PE 1 - PUT: nvshmemx_putmem_block of `bytes`
 * of data + quiet (afterwards PE 1's data equals PE 0's); GET: nvshmemx_getmem_block (PE 0's data
 * equals PE 1's); P: nvshmem_uint64_p(sig, i) + quiet (PE 1's sig[0] == iters); G: nvshmem_uint64_g
 * of PE 1's sig[0], the sum of the values read goes to PE 0's sig[1]; ATOMIC: a dependent chain of
 * nvshmem_uint64_atomic_fetch_add(sig, 1) (PE 1's sig[0] grows by iters, the last value fetched
 * goes to PE 0's sig[1]).  Kinds 5-7: PE 0 and PE 1 bounce a word with signal_op SET / uint64_p /
 * atomic_inc and nvshmem_uint64_wait_until(EQ): sig[0] must be 0 before, is iters on both after.
 * sig holds two words per PE; npes must be >= 2. */
enum {
    NVSHMEM_PERFTEST_LAT_PUT = 0,
    NVSHMEM_PERFTEST_LAT_GET = 1,
    NVSHMEM_PERFTEST_LAT_P = 2,
    NVSHMEM_PERFTEST_LAT_G = 3,
    NVSHMEM_PERFTEST_LAT_ATOMIC = 4,
    NVSHMEM_PERFTEST_LAT_SIGNAL_PINGPONG = 5,
    NVSHMEM_PERFTEST_LAT_P_PINGPONG = 6,
    NVSHMEM_PERFTEST_LAT_ATOMIC_PINGPONG = 7
};
int nvshmem_perftest_pt2pt_latency(int what, void *data, uint64_t *sig, size_t bytes, int iters,
                                   int threads, void *stream);

/* Element-wise bandwidth kernels in the shape of perftest/device/pt-to-pt/shmem_p_bw.cu:43-84,
 * shmem_g_bw.cu, shmem_st_bw.cu and shmem_atomic_bw.cu: every thread handles single elements of
 * elem_bytes (1, 2, 4 or 8; ADD: 4 or 8), consecutive threads consecutive elements, grid-stride over
 * nelems.  P: nvshmem_<uintN>_p(dest + i, src[i], right neighbour); G: dest[i] = nvshmem_<uintN>_g(src
 * + i, right neighbour); ST: the same as P by a plain store through nvshmem_ptr; ADD:
 * nvshmem_<uintN>_atomic_add(dest + i, src[i], right neighbour).  After P / ST / ADD PE p's dest holds
 * (ADD: has grown by) PE p-1's src, after G PE p+1's. */
enum {
    NVSHMEM_PERFTEST_ELEMENT_P = 0,
    NVSHMEM_PERFTEST_ELEMENT_G = 1,
    NVSHMEM_PERFTEST_ELEMENT_ST = 2,
    NVSHMEM_PERFTEST_ELEMENT_ADD = 3
};
int nvshmem_perftest_element_bw(int what, int elem_bytes, void *dest, const void *src, size_t nelems,
                                int blocks_per_pe, int threads, void *stream);

/* Ring allreduce of int32 built from put_signal_nbi + signal_wait_until, the algorithm of
 * examples/ring-reduce.cu:88-144: reduce phase around the ring, then broadcast phase.  nreduce must
 * be a multiple of blocks*chunk_elems.  signal holds `blocks` words (zero before the call; the
 * kernel zeroes them again).  Known answer of the example: src[i]=i on all PEs => dst[i]=i*npes. */
int nvshmem_perftest_ring_reduce(int32_t *dst, const int32_t *src, size_t nreduce,
                                 uint64_t *signal, size_t chunk_elems, int blocks, int threads,
                                 void *stream);

/* Walks through typed / sized / strided RMA in all scopes, scalar p/g, thread-scope put_signal,
 * typed wait / test and sync_all on small fixed layouts (a, b: 8 KiB; sig: 4 words, zero before
 * the call; ints: 8 int32, zero; out: 16 int64).  tests/test_gpu_api_matrix.py states what each
 * region must hold afterwards. */
int nvshmem_perftest_api_matrix(void *a, void *b, uint64_t *sig, int *ints, int64_t *out,
                                int threads, void *stream);

/* In-kernel collectives, one thread group per PE (grid 1 x 1 x npes).  dtype/op use the numbering
 * of nvshmemi_amd_dtype_t / nvshmemi_amd_op_t; supported pairs: (i32,sum) (i64,xor) (f32,sum)
 * (f32,max) (bf16,sum) (bf16,max) (u64,and) (f64,prod) (i16,min).  Returns NOT_SUPPORTED else. */
/* 1 if the in-kernel collective kernels of the library were built with NVSHMEMI_AMD_UNIT_PACKETS (the 64-byte
 * line packets of the small allreduce / reducescatter; libnvshmem_amd_perftest_units.so is), else 0. */
int nvshmem_perftest_unit_packets_compiled(void);
int nvshmem_perftest_device_reduce(int dtype, int op, void *dest, const void *src, size_t nreduce,
                                   int scope, int threads, void *stream);
int nvshmem_perftest_device_fcollect(void *dest, const void *src, size_t bytes, int scope,
                                     int threads, void *stream);
int nvshmem_perftest_device_alltoall(void *dest, const void *src, size_t bytes, int scope,
                                     int threads, void *stream);
/* reducescatter: src holds npes blocks of nreduce elements, dest nreduce elements; supported pairs:
 * (i32,sum) (f32,sum) (f32,max) (bf16,sum) (u64,xor).  broadcast: `bytes` from PE root's src into
 * every PE's dest. */
int nvshmem_perftest_device_reducescatter(int dtype, int op, void *dest, const void *src,
                                          size_t nreduce, int scope, int threads, void *stream);
int nvshmem_perftest_device_broadcast(void *dest, const void *src, size_t bytes, int root,
                                      int scope, int threads, void *stream);
/* Atomic memory operations.  amo_matrix: every PE applies every stamped (type, operation) pair once
 * to word k of `slots` on its right neighbour - case order: fetch, set, swap for the standard then
 * the extended types; compare_swap, compare_swap, fetch_add, add, fetch_inc, inc for the standard
 * types; fetch_and, and, fetch_or, or, fetch_xor, xor for the bitwise types (type lists of
 * include/nvshmem_amd/nvshmem_types.h) - with operands val[k] / cond[k] from its own copies, and
 * stores the returned value into its out[k]; *ncases receives the number of cases, which
 * nvshmem_perftest_amo_matrix_cases() also returns.  All arrays are symmetric, cases + 1 words. */
int nvshmem_perftest_amo_matrix_cases(void);
int nvshmem_perftest_amo_matrix(uint64_t *slots, const uint64_t *val, const uint64_t *cond,
                                uint64_t *out, int *ncases, void *stream);
/* All blocks x threads x npes threads contend for PE `home`'s copies of words[0..8) = {ticket
 * counter, lock, xor word, or word, and word, 32-bit sum, swap word, lock winners} and seen[ticket];
 * chain[id] on PE `home` (symmetric, one word per thread) receives what the thread's swap
 * returned. */
int nvshmem_perftest_amo_contend(uint64_t *words, unsigned int *seen, unsigned long long *chain,
                                 int home, int blocks, int threads, void *stream);
/* `rounds` rounds of {int32 sum reduce of n elements, broadcast of those n elements from PE
 * r % npes, fcollect of fc_bytes (a multiple of 4, at most 4n) per PE, and when n >= npes an
 * alltoall and an int32 sum reducescatter of n / npes words per member} back to back inside one
 * kernel, all on NVSHMEM_TEAM_WORLD into dst, with no barrier in between unless sync_between is
 * set.  Round r sends src[i] = (me*1000003 + r*7919 + i*31) & 0x7fffffff.  After every collective
 * each PE folds dst into its check[0]: h = h*1000003 + sum_i (uint32)dst[i] * (2i+1) (mod 2^64),
 * over the n (reduce, broadcast), fc_bytes*npes/4 (fcollect), (n/npes)*npes (alltoall) or n/npes
 * (reducescatter) words the call produced. */
int nvshmem_perftest_coll_sequence(int32_t *src, int32_t *dst, uint64_t *check, int n, int fc_bytes,
                                   int rounds, int sync_between, int scope, int threads, void *stream);
/* In-kernel collectives on a team handle (members only; the other PEs return at once).  what:
 * 0 float sum reduce (n elements), 1 float sum reducescatter (n per member), 2 fcollectmem, 3
 * alltoallmem, 4 broadcastmem from member `root` (n bytes). */
int nvshmem_perftest_device_team_coll(int what, int team, void *dest, const void *src, size_t n,
                                      int root, int scope, int threads, void *stream);
/* The same call repeated `iters` times inside one kernel (the launch is paid once), for latency
 * measurements; what = 5 adds nvshmem_barrier(team), what = 6 nvshmem_team_sync(team). */
int nvshmem_perftest_device_team_coll_loop(int what, int team, void *dest, const void *src,
                                           size_t n, int root, int iters, int scope, int threads,
                                           void *stream);
/* One block of `threads` per PE calls nvshmemx_double2_maxloc_reduce_block(team, dest, src, nreduce)
 * `iters` times (perftest/device/coll/redmaxloc_latency.cu); dest and src hold nreduce (value,
 * location) pairs of doubles.  With info != NULL (4 ints, symmetric) thread 0 of every PE also
 * records what the device-side nvshmem_info_get_version, nvshmemx_vendor_get_version_info
 * (major * 10000 + minor * 100 + patch) and nvshmem_info_get_name (length of the name) report. */
int nvshmem_perftest_device_maxloc(int team, void *dest, const void *src, size_t nreduce, int iters,
                                   int threads, int *info, void *stream);

/* Every PE writes into its copy of `out` (4 + 64 ints): team_my_pe(a), team_n_pes(a),
 * team_my_pe(b), team_n_pes(b), then team_translate_pe(a, i, b) for i = 0..63, all evaluated in
 * device code. */
int nvshmem_perftest_team_query(int *out, int team_a, int team_b, void *stream);
/* device_barrier among the members of `team` (nvshmem_barrier(team) / nvshmem_team_sync(team)). */
int nvshmem_perftest_device_team_barrier(uint64_t *counter, uint64_t *errors, int rounds, int team,
                                         int scope, int threads, void *stream);
/* The same rounds run by ONE warpgroup of every member through nvshmemx_barrier_warpgroup: warpgroup
 * `group` = threads [256 group, 256 group + 256) of the one block per PE (the last group may be
 * shorter); the block's other threads leave at once. */
int nvshmem_perftest_device_warpgroup_barrier(uint64_t *counter, uint64_t *errors, int rounds, int team,
                                              int group, int threads, void *stream);
/* `rounds` barriers; before round r each PE stores r into its `counter`, after the barrier it reads
 * every PE's counter and adds to its own errors[0] the number that are < r.  counter and errors
 * hold one uint64 each. */
int nvshmem_perftest_device_barrier(uint64_t *counter, uint64_t *errors, int rounds, int scope,
                                    int threads, void *stream);

/*
 * MoE token shuffle (config: npes PEs, `tokens` rows of `row_bytes` per PE, `topk` copies per
 * token).  Routing tables are device arrays in symmetric memory, one copy per PE, filled by the
 * caller:  dest_pe[t*topk+k] (int32) and dest_row[t*topk+k] (int64) say where copy k of token t
 * lands; expected[src] (uint64, npes words) is the number of rows this PE receives from PE src.
 *   dispatch: recv@dest_pe[dest_row] = send[t]   via nvshmemx_putmem_signal_nbi_block with
 *             NVSHMEM_SIGNAL_ADD of 1 on sig[src] at the destination; then every PE waits until
 *             sig[src] >= expected[src] for all src (nvshmem_signal_wait_until, CMP_GE).
 *   combine:  out[t*topk+k] = recv@dest_pe[dest_row]  via nvshmemx_getmem_nbi_block.
 * sig holds npes words per PE and must be zero before dispatch.  recv holds recv_cap_rows rows on
 * every PE; a routing entry outside [0, npes) x [0, recv_cap_rows) is skipped.  blocks_per_pe
 * blocks of `threads` threads per PE; dispatch is a cooperative launch (it waits on other PEs).
 * The plain entry points move one row per wavefront and publish one signal update per block and
 * destination; the _ex forms choose the scope (NVSHMEM_PERFTEST_SCOPE_WARP or _BLOCK) and, with
 * bit 8 set in `scope` (dispatch only), signal after every row with nvshmemx_putmem_signal_nbi_warp /
 * _block, the put_signal_nbi + signal_wait_until(GE) idiom of examples/ring-reduce.cu:111-127; bit 9
 * on top of it gives those signals the NVSHMEMX_AMD_SIGNAL_PAYLOAD_ONLY ordering.  _put_signal is the
 * _ex form with the signal word of source PE s at sig[s * sig_stride] (sig then holds npes *
 * sig_stride words per PE): atomic updates of one 128-byte line are applied one after the other at
 * about 80 ns each, so per-row signals from eight sources into one line take longer than the rows.
 */
int nvshmem_perftest_moe_dispatch(void *recv, size_t recv_cap_rows, const void *send,
                                  const int32_t *dest_pe, const int64_t *dest_row,
                                  const uint64_t *expected, uint64_t *sig, int tokens, int topk,
                                  size_t row_bytes, int blocks_per_pe, int threads, void *stream);
int nvshmem_perftest_moe_dispatch_ex(void *recv, size_t recv_cap_rows, const void *send,
                                     const int32_t *dest_pe, const int64_t *dest_row,
                                     const uint64_t *expected, uint64_t *sig, int tokens, int topk,
                                     size_t row_bytes, int blocks_per_pe, int threads, int scope,
                                     void *stream);
int nvshmem_perftest_moe_dispatch_put_signal(void *recv, size_t recv_cap_rows, const void *send,
                                             const int32_t *dest_pe, const int64_t *dest_row,
                                             const uint64_t *expected, uint64_t *sig, int sig_stride,
                                             int tokens, int topk, size_t row_bytes, int blocks_per_pe,
                                             int threads, int scope, void *stream);
int nvshmem_perftest_moe_combine(void *out, const void *recv, size_t recv_cap_rows,
                                 const int32_t *dest_pe, const int64_t *dest_row, int tokens,
                                 int topk, size_t row_bytes, int blocks_per_pe, int threads,
                                 void *stream);
int nvshmem_perftest_moe_combine_ex(void *out, const void *recv, size_t recv_cap_rows,
                                    const int32_t *dest_pe, const int64_t *dest_row, int tokens,
                                    int topk, size_t row_bytes, int blocks_per_pe, int threads,
                                    int scope, void *stream);
/* Dispatch as two launches on `stream`: a grid with one wavefront per work item - piece_bytes (1024,
 * 2048 or 4096) of one token's row, pushed to all of its topk destinations - then one block per PE
 * that publishes the row counts through the signal words and waits for the expected ones.  A block of
 * `threads` (a multiple of 64) takes threads / 64 tokens.  With 16-byte aligned buffers and rows the
 * piece is loaded once and stored through nvshmem_ptr; otherwise (or when the environment variable
 * NVSHMEM_PERFTEST_MOE_PUTS is set) it is moved with topk nvshmemx_putmem_nbi_warp calls. */
int nvshmem_perftest_moe_dispatch_pieces(void *recv, size_t recv_cap_rows, const void *send,
                                         const int32_t *dest_pe, const int64_t *dest_row,
                                         const uint64_t *expected, uint64_t *sig, int tokens, int topk,
                                         size_t row_bytes, int piece_bytes, int threads, void *stream);
/* nvshmem_perftest_moe_dispatch_pieces for callers that cannot allocate (code under HIP graph capture,
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  It takes no signal
 * words from the caller: they live in a static device array of the library (8 KiB per GPU, rows for at
 * most 32 PEs; more PEs are refused with NVSHMEMX_ERROR_INVALID_VALUE and a message), which a kernel on
 * `stream` clears before the rows are sent.  It calls no hipMalloc, hipFree or other allocating routine.
 * All calls on one GPU share that array: calls that overlap in time on one GPU race (two host threads
 * inside the call at once are refused; kernels of calls on different streams that overlap on the GPU are
 * the caller's to avoid).  The array's address is looked up once per GPU, in nvshmem_perftest_static_init()
 * or in the first call on that GPU; under stream capture no lookup is made, so a caller that captures its
 * first call runs nvshmem_perftest_static_init() beforehand, with that GPU current. */
int nvshmem_perftest_static_init(void);
int nvshmem_perftest_moe_dispatch_pieces_static(void *recv, size_t recv_cap_rows, const void *send,
                                                const int32_t *dest_pe, const int64_t *dest_row,
                                                const uint64_t *expected, int tokens, int topk,
                                                size_t row_bytes, int piece_bytes, int threads,
                                                void *stream);
/* The same with a work item of piece_bytes (1024, 2048 or 4096; wavefront scope) of a row instead of
 * a whole row (0): with 2 KiB items and one wavefront per block every block moves one short piece
 * and exits. */
int nvshmem_perftest_moe_combine_pieces(void *out, const void *recv, size_t recv_cap_rows,
                                        const int32_t *dest_pe, const int64_t *dest_row, int tokens,
                                        int topk, size_t row_bytes, int piece_bytes,
                                        int blocks_per_pe, int threads, int scope, void *stream);
/* Per-expert counts exchange + prefix sum on the device (examples/moe_shuffle.cu:204-234):
 * counts holds num_experts int64 per PE (rows this PE sends to each expert); on return
 * seg_base[e*npes + src] (int64, num_experts*npes words per PE, every PE gets the full table) is the
 * first receive row of segment (expert e, source src) and recv_rows[0] the rows this PE receives. */
int nvshmem_perftest_moe_exchange_offsets(const int64_t *counts, int64_t *seg_base,
                                          int64_t *recv_rows, int num_experts, void *stream);

#ifdef __cplusplus
}
#endif
#endif
