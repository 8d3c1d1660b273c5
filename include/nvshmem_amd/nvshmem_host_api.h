/*
 * Host C ABI of libnvshmem_amd.so: the entry points a caller of the reference's host library binds
 * for the data-movement path.  Plain C types only; a stream is an opaque `void *` holding a
 * hipStream_t (NULL = the null stream).
 *
 * Execution model.  All PEs are logical: one process, one GPU, one hipMalloc'd heap cut into npes
 * equal power-of-two slices.  The host thread stands for the whole SPMD program ("collapsed SPMD"):
 *   - a symmetric pointer returned by nvshmem_malloc is the address of the object in PE 0's slice
 *     (its canonical address); nvshmem_ptr(p, pe) gives the address of PE pe's copy;
 *   - one call of a collective performs it for every PE of the team (the reference needs one call
 *     per PE process); nvshmem_my_pe() on the host is 0;
 *   - point-to-point host calls act as PE 0 unless a source/dest pointer obtained from
 *     nvshmem_ptr(x, q) names another PE's copy explicitly.
 *
 * Each declaration cites the reference declaration it replaces (paths under the reference tree).
 */
#ifndef NVSHMEM_AMD_HOST_API_H
#define NVSHMEM_AMD_HOST_API_H

#include "nvshmem_types.h"

#if defined(__HIPCC__)
#define NVSHMEMI_HOST_ONLY __host__
#else
#define NVSHMEMI_HOST_ONLY
#endif

#ifdef __cplusplus
extern "C" {
#endif

typedef void *nvshmemx_stream_t; /* hipStream_t */

/* ---- library setup: src/include/host/nvshmem_api.h:50-88 ---- */
NVSHMEMI_HOST_ONLY void nvshmem_init(void);           /* nvshmem_api.h:52-58 */
NVSHMEMI_HOST_ONLY void nvshmem_finalize(void);       /* nvshmem_api.h:66 */
NVSHMEMI_HOST_ONLY int nvshmemx_init_status(void);    /* nvshmem_api.h:50 */
/* nvshmem_init with a thread level (nvshmem_api.h:60-67); `provided` is NVSHMEM_THREAD_SERIALIZED
 * whatever was requested, as in the reference (src/host/init/init.cu:1294,1309).  Returns 0. */
NVSHMEMI_HOST_ONLY int nvshmem_init_thread(int requested, int *provided);
NVSHMEMI_HOST_ONLY void nvshmem_query_thread(int *provided);   /* nvshmem_api.h:69 */
/* Ends the program with `status` after finalizing (nvshmem_api.h:70). */
NVSHMEMI_HOST_ONLY void nvshmem_global_exit(int status);
/* Registration of local buffers used as put sources / get destinations
 * (src/include/host/nvshmemx_api.h:47-49): every device allocation of the one GPU is reachable by
 * load/store already, so these only validate their arguments and return 0. */
NVSHMEMI_HOST_ONLY int nvshmemx_buffer_register(void *addr, size_t length);
NVSHMEMI_HOST_ONLY int nvshmemx_buffer_unregister(void *addr);
NVSHMEMI_HOST_ONLY void nvshmemx_buffer_unregister_all(void);
NVSHMEMI_HOST_ONLY int nvshmem_my_pe(void);           /* nvshmem_api.h:60-64 */
NVSHMEMI_HOST_ONLY int nvshmem_n_pes(void);
/* ---- teams: src/include/host/nvshmem_api.h:465-482, src/host/team/team.cu:19-115 ----
 * A team is a strided set of world PEs.  The host thread stands for every PE, so one split call
 * creates the team for all of its members, and a handle can name a family of disjoint teams: after
 * nvshmem_team_split_2d the x handle is "my row" and the y handle "my column" for every PE, as the
 * variables of the same names are in an SPMD program.  A collective called on such a handle runs on
 * every team of the family.  Queries without a PE argument answer for PE 0 (the host's
 * nvshmem_my_pe()); nvshmemx_amd_team_view answers for any PE.  Handles are small integers that
 * are reused after nvshmem_team_destroy; at most NVSHMEMI_AMD_MAX_TEAMS exist at a time. */
NVSHMEMI_HOST_ONLY int nvshmem_team_my_pe(nvshmem_team_t team); /* nvshmem_api.h:465 */
NVSHMEMI_HOST_ONLY int nvshmem_team_n_pes(nvshmem_team_t team); /* nvshmem_api.h:466 */
NVSHMEMI_HOST_ONLY void nvshmem_team_get_config(nvshmem_team_t team,
                                                nvshmem_team_config_t *config); /* :468 */
NVSHMEMI_HOST_ONLY int nvshmem_team_translate_pe(nvshmem_team_t src_team, int src_pe,
                                                 nvshmem_team_t dest_team); /* :469 */
/* Members PE_start, PE_start + PE_stride, ... (PE_size of them) of the parent, counted in parent
 * indices, in every team of the parent's family; the others are not members of the new handle.
 * Returns 0 and the handle, or nonzero and NVSHMEM_TEAM_INVALID (argument errors of
 * team_internal.cpp:2197-2222, or no free handle). */
NVSHMEMI_HOST_ONLY int nvshmem_team_split_strided(nvshmem_team_t parent_team, int PE_start,
                                                  int PE_stride, int PE_size,
                                                  const nvshmem_team_config_t *config,
                                                  long config_mask,
                                                  nvshmem_team_t *new_team); /* :471 */
/* Row-major grid with rows of xrange members (team_internal.cpp:2292-2349): *xaxis_team names
 * every PE's row, *yaxis_team every PE's column. */
NVSHMEMI_HOST_ONLY int nvshmem_team_split_2d(nvshmem_team_t parent_team, int xrange,
                                             const nvshmem_team_config_t *xaxis_config,
                                             long xaxis_mask, nvshmem_team_t *xaxis_team,
                                             const nvshmem_team_config_t *yaxis_config,
                                             long yaxis_mask,
                                             nvshmem_team_t *yaxis_team); /* :478 */
NVSHMEMI_HOST_ONLY void nvshmem_team_destroy(nvshmem_team_t team); /* :482 */
/* {start, stride, size, my_pe} of `team` as world PE `pe` sees it (size 0: not a member).
 * Returns 0, or NVSHMEMX_ERROR_INVALID_VALUE for a handle or PE that does not exist. */
NVSHMEMI_HOST_ONLY int nvshmemx_amd_team_view(nvshmem_team_t team, int pe, int view[4]);
NVSHMEMI_HOST_ONLY void nvshmem_info_get_version(int *major, int *minor); /* nvshmem_api.h:77 */
NVSHMEMI_HOST_ONLY void nvshmem_info_get_name(char *name);                /* nvshmem_api.h:78 */
NVSHMEMI_HOST_ONLY void nvshmemx_vendor_get_version_info(int *major, int *minor, int *patch);

/*
 * Logical-PE bring-up (stands where the reference's nvshmemx_init_attr + bootstrap sit,
 * src/include/host/nvshmemx_api.h:52-66): npes PEs with symmetric_size bytes each (the distance
 * between two PEs' slices is that size plus 2 KiB of runtime words, rounded up to 16 MiB, or to 2 MiB for
 * heaps of at most 16 MiB).  nvshmem_init() calls it with NVSHMEM_AMD_NPES (default 8) and
 * NVSHMEM_SYMMETRIC_SIZE (default 1 GiB; reference src/include/host/env/env_defs.h).
 * Returns an nvshmemx_status.
 */
NVSHMEMI_HOST_ONLY int nvshmemx_amd_init(int npes, size_t symmetric_size);

/* ---- symmetric heap: src/include/host/nvshmem_api.h:83-88, src/host/mem/mem_heap.cpp:2288-2387 ---- */
NVSHMEMI_HOST_ONLY void *nvshmem_malloc(size_t size);
NVSHMEMI_HOST_ONLY void *nvshmem_calloc(size_t count, size_t size);
NVSHMEMI_HOST_ONLY void *nvshmem_align(size_t alignment, size_t size);
NVSHMEMI_HOST_ONLY void nvshmem_free(void *ptr);
NVSHMEMI_HOST_ONLY void *nvshmem_ptr(const void *ptr, int pe);

/* ---- ordering and barriers: nvshmem_api.h:359-461, nvshmem_coll_api.h:41-48 ---- */
NVSHMEMI_HOST_ONLY void nvshmem_quiet(void);
NVSHMEMI_HOST_ONLY void nvshmem_fence(void);
NVSHMEMI_HOST_ONLY void nvshmem_barrier_all(void);
NVSHMEMI_HOST_ONLY int nvshmem_barrier(nvshmem_team_t team);
NVSHMEMI_HOST_ONLY void nvshmem_sync_all(void);
NVSHMEMI_HOST_ONLY int nvshmem_team_sync(nvshmem_team_t team);
/* src/include/host/nvshmemx_coll_api.h:36-41, nvshmemx_api.h:250 */
NVSHMEMI_HOST_ONLY void nvshmemx_barrier_all_on_stream(nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY int nvshmemx_barrier_on_stream(nvshmem_team_t team, nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY void nvshmemx_sync_all_on_stream(nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY int nvshmemx_team_sync_on_stream(nvshmem_team_t team, nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY void nvshmemx_quiet_on_stream(nvshmemx_stream_t stream);

/* ---- host-initiated RMA: nvshmem_api.h:199-353 (blocking), nvshmemx_api.h:94-248 (on stream) ---- */
NVSHMEMI_HOST_ONLY void nvshmem_putmem(void *dest, const void *source, size_t bytes, int pe);
NVSHMEMI_HOST_ONLY void nvshmem_getmem(void *dest, const void *source, size_t bytes, int pe);
NVSHMEMI_HOST_ONLY void nvshmem_putmem_nbi(void *dest, const void *source, size_t bytes, int pe);
NVSHMEMI_HOST_ONLY void nvshmem_getmem_nbi(void *dest, const void *source, size_t bytes, int pe);
NVSHMEMI_HOST_ONLY void nvshmemx_putmem_on_stream(void *dest, const void *source, size_t bytes,
                                                  int pe, nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY void nvshmemx_getmem_on_stream(void *dest, const void *source, size_t bytes,
                                                  int pe, nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY void nvshmemx_putmem_nbi_on_stream(void *dest, const void *source, size_t bytes,
                                                      int pe, nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY void nvshmemx_getmem_nbi_on_stream(void *dest, const void *source, size_t bytes,
                                                      int pe, nvshmemx_stream_t stream);
/* nvshmemx_api.h:133-136, :153-156 */
NVSHMEMI_HOST_ONLY void nvshmemx_putmem_signal_on_stream(void *dest, const void *source,
                                                         size_t bytes, uint64_t *sig_addr,
                                                         uint64_t signal, int sig_op, int pe,
                                                         nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY void nvshmemx_putmem_signal_nbi_on_stream(void *dest, const void *source,
                                                             size_t bytes, uint64_t *sig_addr,
                                                             uint64_t signal, int sig_op, int pe,
                                                             nvshmemx_stream_t stream);
/* nvshmemx_api.h:252-253, :275-276; host kernels src/include/internal/non_abi/nvshmemi_h_to_d_sync_defs.cuh:72-90 */
NVSHMEMI_HOST_ONLY void nvshmemx_signal_op_on_stream(uint64_t *sig_addr, uint64_t signal,
                                                     int sig_op, int pe, nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY void nvshmemx_signal_wait_until_on_stream(uint64_t *sig_addr, int cmp,
                                                             uint64_t cmp_value,
                                                             nvshmemx_stream_t stream);

/* typed forms: nvshmem_api.h:199-306 (blocking), nvshmemx_api.h:94-248 (on stream).  p takes the
 * value in the call, g returns it (and therefore waits for the stream).  iput / iget: element i of
 * the source at stride sst goes to element i*dst of the destination; strides are at least 1. */
#define NVSHMEMI_DECL_TYPED_RMA_HOST(NAME, TYPE, TAG)                                             \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_put(TYPE *dest, const TYPE *source, size_t nelems,   \
                                                 int pe);                                         \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_get(TYPE *dest, const TYPE *source, size_t nelems,   \
                                                 int pe);                                         \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_put_nbi(TYPE *dest, const TYPE *source,              \
                                                     size_t nelems, int pe);                      \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_get_nbi(TYPE *dest, const TYPE *source,              \
                                                     size_t nelems, int pe);                      \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_p(TYPE *dest, const TYPE value, int pe);             \
    NVSHMEMI_HOST_ONLY TYPE nvshmem_##NAME##_g(const TYPE *src, int pe);                          \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_iput(TYPE *dest, const TYPE *source, ptrdiff_t dst,  \
                                                  ptrdiff_t sst, size_t nelems, int pe);          \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_iget(TYPE *dest, const TYPE *source, ptrdiff_t dst,  \
                                                  ptrdiff_t sst, size_t nelems, int pe);          \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_put_on_stream(                                      \
        TYPE *dest, const TYPE *source, size_t nelems, int pe, nvshmemx_stream_t stream);         \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_get_on_stream(                                      \
        TYPE *dest, const TYPE *source, size_t nelems, int pe, nvshmemx_stream_t stream);         \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_put_nbi_on_stream(                                  \
        TYPE *dest, const TYPE *source, size_t nelems, int pe, nvshmemx_stream_t stream);         \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_get_nbi_on_stream(                                  \
        TYPE *dest, const TYPE *source, size_t nelems, int pe, nvshmemx_stream_t stream);         \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_p_on_stream(TYPE *dest, const TYPE value, int pe,   \
                                                          nvshmemx_stream_t stream);              \
    NVSHMEMI_HOST_ONLY TYPE nvshmemx_##NAME##_g_on_stream(const TYPE *src, int pe,                \
                                                          nvshmemx_stream_t stream);              \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_iput_on_stream(                                     \
        TYPE *dest, const TYPE *source, ptrdiff_t dst, ptrdiff_t sst, size_t nelems, int pe,      \
        nvshmemx_stream_t stream);                                                                \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_iget_on_stream(                                     \
        TYPE *dest, const TYPE *source, ptrdiff_t dst, ptrdiff_t sst, size_t nelems, int pe,      \
        nvshmemx_stream_t stream);                                                                \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_put_signal_on_stream(                               \
        TYPE *dest, const TYPE *source, size_t nelems, uint64_t *sig_addr, uint64_t signal,       \
        int sig_op, int pe, nvshmemx_stream_t stream);                                            \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_put_signal_nbi_on_stream(                           \
        TYPE *dest, const TYPE *source, size_t nelems, uint64_t *sig_addr, uint64_t signal,       \
        int sig_op, int pe, nvshmemx_stream_t stream);
NVSHMEMI_REPT_FOR_STANDARD_RMA_TYPES(NVSHMEMI_DECL_TYPED_RMA_HOST)
#undef NVSHMEMI_DECL_TYPED_RMA_HOST

/* sized forms put8 .. put128: nelems elements of BITS/8 bytes (nvshmem_api.h:214-306,
 * nvshmemx_api.h:106-248) */
#define NVSHMEMI_DECL_SIZED_RMA_HOST(BITS, BYTES)                                                 \
    NVSHMEMI_HOST_ONLY void nvshmem_put##BITS(void *dest, const void *source, size_t nelems,      \
                                              int pe);                                            \
    NVSHMEMI_HOST_ONLY void nvshmem_get##BITS(void *dest, const void *source, size_t nelems,      \
                                              int pe);                                            \
    NVSHMEMI_HOST_ONLY void nvshmem_put##BITS##_nbi(void *dest, const void *source,               \
                                                    size_t nelems, int pe);                       \
    NVSHMEMI_HOST_ONLY void nvshmem_get##BITS##_nbi(void *dest, const void *source,               \
                                                    size_t nelems, int pe);                       \
    NVSHMEMI_HOST_ONLY void nvshmem_iput##BITS(void *dest, const void *source, ptrdiff_t dst,     \
                                               ptrdiff_t sst, size_t nelems, int pe);             \
    NVSHMEMI_HOST_ONLY void nvshmem_iget##BITS(void *dest, const void *source, ptrdiff_t dst,     \
                                               ptrdiff_t sst, size_t nelems, int pe);             \
    NVSHMEMI_HOST_ONLY void nvshmemx_put##BITS##_on_stream(void *dest, const void *source,        \
                                                           size_t nelems, int pe,                 \
                                                           nvshmemx_stream_t stream);             \
    NVSHMEMI_HOST_ONLY void nvshmemx_get##BITS##_on_stream(void *dest, const void *source,        \
                                                           size_t nelems, int pe,                 \
                                                           nvshmemx_stream_t stream);             \
    NVSHMEMI_HOST_ONLY void nvshmemx_put##BITS##_nbi_on_stream(void *dest, const void *source,    \
                                                               size_t nelems, int pe,             \
                                                               nvshmemx_stream_t stream);         \
    NVSHMEMI_HOST_ONLY void nvshmemx_get##BITS##_nbi_on_stream(void *dest, const void *source,    \
                                                               size_t nelems, int pe,             \
                                                               nvshmemx_stream_t stream);         \
    NVSHMEMI_HOST_ONLY void nvshmemx_iput##BITS##_on_stream(void *dest, const void *source,       \
                                                            ptrdiff_t dst, ptrdiff_t sst,         \
                                                            size_t nelems, int pe,                \
                                                            nvshmemx_stream_t stream);            \
    NVSHMEMI_HOST_ONLY void nvshmemx_iget##BITS##_on_stream(void *dest, const void *source,       \
                                                            ptrdiff_t dst, ptrdiff_t sst,         \
                                                            size_t nelems, int pe,                \
                                                            nvshmemx_stream_t stream);            \
    NVSHMEMI_HOST_ONLY void nvshmemx_put##BITS##_signal_on_stream(                                \
        void *dest, const void *source, size_t nelems, uint64_t *sig_addr, uint64_t signal,       \
        int sig_op, int pe, nvshmemx_stream_t stream);                                            \
    NVSHMEMI_HOST_ONLY void nvshmemx_put##BITS##_signal_nbi_on_stream(                            \
        void *dest, const void *source, size_t nelems, uint64_t *sig_addr, uint64_t signal,       \
        int sig_op, int pe, nvshmemx_stream_t stream);
NVSHMEMI_REPT_FOR_SIZES(NVSHMEMI_DECL_SIZED_RMA_HOST)
#undef NVSHMEMI_DECL_SIZED_RMA_HOST

/* typed waits on a stream (nvshmemx_api.h:255-273): a one-block kernel that spins (bounded by the
 * spin limit) on the local word(s); `status` is device-accessible or NULL.  nvshmem_signal_fetch
 * (nvshmem_api.h:343) reads the calling PE's signal word. */
#define NVSHMEMI_DECL_WAIT_ON_STREAM(NAME, TYPE)                                                  \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_wait_until_on_stream(TYPE *ivar, int cmp,           \
                                                                   TYPE cmp_value,                \
                                                                   nvshmemx_stream_t stream);     \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_wait_until_all_on_stream(                           \
        TYPE *ivars, size_t nelems, const int *status, int cmp, TYPE cmp_value,                   \
        nvshmemx_stream_t stream);                                                                \
    NVSHMEMI_HOST_ONLY void nvshmemx_##NAME##_wait_until_all_vector_on_stream(                    \
        TYPE *ivars, size_t nelems, const int *status, int cmp, TYPE *cmp_values,                 \
        nvshmemx_stream_t stream);
NVSHMEMI_REPT_FOR_WAIT_TYPES(NVSHMEMI_DECL_WAIT_ON_STREAM)
#undef NVSHMEMI_DECL_WAIT_ON_STREAM
NVSHMEMI_HOST_ONLY uint64_t nvshmem_signal_fetch(uint64_t *sig_addr);

/* ---- atomic memory operations from the host (nvshmem_api.h:113-197) ----
 * Blocking: the operation is applied to `target` on PE `pe` by a one-thread kernel on the default
 * stream and the call returns once it is done (with the value fetched, for the fetching forms).
 * The reference declares the same names and defines them as stubs that print "not implemented"
 * (src/host/comm/amo.cpp); here they perform the operation. */
#define NVSHMEMI_DECL_AMO_FETCH_SET_SWAP_HOST(NAME, TYPE)                                         \
    NVSHMEMI_HOST_ONLY TYPE nvshmem_##NAME##_atomic_fetch(const TYPE *target, int pe);            \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_atomic_set(TYPE *target, TYPE value, int pe);        \
    NVSHMEMI_HOST_ONLY TYPE nvshmem_##NAME##_atomic_swap(TYPE *target, TYPE value, int pe);
NVSHMEMI_REPT_FOR_STANDARD_AMO_TYPES(NVSHMEMI_DECL_AMO_FETCH_SET_SWAP_HOST)
NVSHMEMI_REPT_FOR_EXTENDED_AMO_TYPES(NVSHMEMI_DECL_AMO_FETCH_SET_SWAP_HOST)
#undef NVSHMEMI_DECL_AMO_FETCH_SET_SWAP_HOST
#define NVSHMEMI_DECL_AMO_ARITH_HOST(NAME, TYPE)                                                  \
    NVSHMEMI_HOST_ONLY TYPE nvshmem_##NAME##_atomic_compare_swap(TYPE *target, TYPE cond,         \
                                                                 TYPE value, int pe);             \
    NVSHMEMI_HOST_ONLY TYPE nvshmem_##NAME##_atomic_fetch_add(TYPE *target, TYPE value, int pe);  \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_atomic_add(TYPE *target, TYPE value, int pe);        \
    NVSHMEMI_HOST_ONLY TYPE nvshmem_##NAME##_atomic_fetch_inc(TYPE *target, int pe);              \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_atomic_inc(TYPE *target, int pe);
NVSHMEMI_REPT_FOR_STANDARD_AMO_TYPES(NVSHMEMI_DECL_AMO_ARITH_HOST)
#undef NVSHMEMI_DECL_AMO_ARITH_HOST
#define NVSHMEMI_DECL_AMO_BITWISE_HOST(NAME, TYPE)                                                \
    NVSHMEMI_HOST_ONLY TYPE nvshmem_##NAME##_atomic_fetch_and(TYPE *target, TYPE value, int pe);  \
    NVSHMEMI_HOST_ONLY TYPE nvshmem_##NAME##_atomic_fetch_or(TYPE *target, TYPE value, int pe);   \
    NVSHMEMI_HOST_ONLY TYPE nvshmem_##NAME##_atomic_fetch_xor(TYPE *target, TYPE value, int pe);  \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_atomic_and(TYPE *target, TYPE value, int pe);        \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_atomic_or(TYPE *target, TYPE value, int pe);         \
    NVSHMEMI_HOST_ONLY void nvshmem_##NAME##_atomic_xor(TYPE *target, TYPE value, int pe);
NVSHMEMI_REPT_FOR_BITWISE_AMO_TYPES(NVSHMEMI_DECL_AMO_BITWISE_HOST)
#undef NVSHMEMI_DECL_AMO_BITWISE_HOST

/* ---- collectives: src/include/host/nvshmem_coll_api.h:27-80, nvshmemx_coll_api.h:27-80 ----
 * One call serves every PE of the team.  dest and src are canonical symmetric addresses.
 * alltoall: dest@j[i*nelems + k] = src@i[j*nelems + k];  fcollect: dest@j[i*nelems + k] = src@i[k];
 * reduce:   dest@j[k] = fold over PEs 0..n-1 in that order of src@i[k];
 * broadcast (nvshmem_coll_api.h:46-54, nvshmemx_coll_api.h:43-52): dest@j[k] = src@PE_root[k] for
 * every PE j of the team, the root included; dest == src is the in-place form;
 * reducescatter (nvshmem_coll_api.h:82-96, nvshmemx_coll_api.h:80-96):
 * dest@j[k] = fold over PEs i = 0..n-1 of src@i[j*nreduce + k]; dest must not overlap src.
 * All return 0 on success. */
#define NVSHMEMI_DECL_TYPED_COLL_HOST(NAME, TYPE, TAG)                                            \
    NVSHMEMI_HOST_ONLY int nvshmem_##NAME##_alltoall(nvshmem_team_t team, TYPE *dest,             \
                                                     const TYPE *src, size_t nelems);             \
    NVSHMEMI_HOST_ONLY int nvshmem_##NAME##_fcollect(nvshmem_team_t team, TYPE *dest,             \
                                                     const TYPE *src, size_t nelems);             \
    NVSHMEMI_HOST_ONLY int nvshmemx_##NAME##_alltoall_on_stream(                                  \
        nvshmem_team_t team, TYPE *dest, const TYPE *src, size_t nelems, nvshmemx_stream_t s);    \
    NVSHMEMI_HOST_ONLY int nvshmemx_##NAME##_fcollect_on_stream(                                  \
        nvshmem_team_t team, TYPE *dest, const TYPE *src, size_t nelems, nvshmemx_stream_t s);    \
    NVSHMEMI_HOST_ONLY int nvshmem_##NAME##_broadcast(nvshmem_team_t team, TYPE *dest,            \
                                                      const TYPE *src, size_t nelems,             \
                                                      int PE_root);                               \
    NVSHMEMI_HOST_ONLY int nvshmemx_##NAME##_broadcast_on_stream(                                 \
        nvshmem_team_t team, TYPE *dest, const TYPE *src, size_t nelems, int PE_root,             \
        nvshmemx_stream_t s);
NVSHMEMI_REPT_FOR_STANDARD_RMA_TYPES(NVSHMEMI_DECL_TYPED_COLL_HOST)
#undef NVSHMEMI_DECL_TYPED_COLL_HOST

NVSHMEMI_HOST_ONLY int nvshmem_alltoallmem(nvshmem_team_t team, void *dest, const void *src,
                                           size_t nelems);
NVSHMEMI_HOST_ONLY int nvshmem_fcollectmem(nvshmem_team_t team, void *dest, const void *src,
                                           size_t nelems);
NVSHMEMI_HOST_ONLY int nvshmem_broadcastmem(nvshmem_team_t team, void *dest, const void *src,
                                            size_t nelems, int PE_root);
NVSHMEMI_HOST_ONLY int nvshmemx_broadcastmem_on_stream(nvshmem_team_t team, void *dest,
                                                       const void *src, size_t nelems,
                                                       int PE_root, nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY int nvshmemx_alltoallmem_on_stream(nvshmem_team_t team, void *dest,
                                                      const void *src, size_t nelems,
                                                      nvshmemx_stream_t stream);
NVSHMEMI_HOST_ONLY int nvshmemx_fcollectmem_on_stream(nvshmem_team_t team, void *dest,
                                                      const void *src, size_t nelems,
                                                      nvshmemx_stream_t stream);

#define NVSHMEMI_DECL_TYPED_REDUCE_HOST(NAME, TYPE, TAG, OP)                                      \
    NVSHMEMI_HOST_ONLY int nvshmem_##NAME##_##OP##_reduce(nvshmem_team_t team, TYPE *dest,        \
                                                          const TYPE *src, size_t nreduce);       \
    NVSHMEMI_HOST_ONLY int nvshmemx_##NAME##_##OP##_reduce_on_stream(                             \
        nvshmem_team_t team, TYPE *dest, const TYPE *src, size_t nreduce, nvshmemx_stream_t s);   \
    NVSHMEMI_HOST_ONLY int nvshmem_##NAME##_##OP##_reducescatter(                                 \
        nvshmem_team_t team, TYPE *dest, const TYPE *src, size_t nreduce);                        \
    NVSHMEMI_HOST_ONLY int nvshmemx_##NAME##_##OP##_reducescatter_on_stream(                      \
        nvshmem_team_t team, TYPE *dest, const TYPE *src, size_t nreduce, nvshmemx_stream_t s);
NVSHMEMI_REPT_FOR_ALL_REDUCE_TYPES_AND_OPS(NVSHMEMI_DECL_TYPED_REDUCE_HOST)
#undef NVSHMEMI_DECL_TYPED_REDUCE_HOST

/*
 * Cooperative launch of a kernel that uses the device API (reference
 * src/device/launch/collective_launch.cpp:209-212).  One launch carries every logical PE:
 * the grid's z extent is set to npes (the caller's grid z must be 1) and a block acts as PE
 * blockIdx.z.  grid (0,0,0) asks for the largest co-resident grid per PE.  The launch is refused
 * with NVSHMEMX_ERROR_COLLECTIVE_LAUNCH_FAILED when grid*npes blocks cannot be co-resident.
 * Grid and block are passed as three unsigned each to keep the ABI free of HIP types.
 */
NVSHMEMI_HOST_ONLY int nvshmemx_amd_collective_launch(const void *func, unsigned grid_x,
                                                      unsigned grid_y, unsigned grid_z,
                                                      unsigned block_x, unsigned block_y,
                                                      unsigned block_z, void **args,
                                                      size_t shared_mem, nvshmemx_stream_t stream);
/* Largest grid.x (blocks per PE) of `func` that nvshmemx_amd_collective_launch accepts
 * (reference nvshmemx_collective_launch_query_gridsize, collective_launch.cpp:214-260). */
NVSHMEMI_HOST_ONLY int nvshmemx_amd_collective_launch_query_gridsize(const void *func,
                                                                     unsigned block_x,
                                                                     unsigned block_y,
                                                                     unsigned block_z,
                                                                     size_t shared_mem,
                                                                     int *gridsize);

/*
 * Registration of a translation unit's copy of the device state.  Every hipcc translation unit that
 * includes the device API holds a private `__constant__` state block and a function that copies a
 * host state block into it; a static initialiser in that unit hands the function to the library,
 * which calls every registered one whenever the state changes (the reference refreshes each
 * registered copy the same way, src/host/init/init.cu:146-197).  The function returns a hipError_t.
 */
typedef int (*nvshmemi_amd_state_updater_t)(const struct nvshmemi_device_state *host_copy);
NVSHMEMI_HOST_ONLY void nvshmemi_amd_register_state_updater(nvshmemi_amd_state_updater_t fn);
NVSHMEMI_HOST_ONLY void nvshmemi_amd_unregister_state_updater(nvshmemi_amd_state_updater_t fn);
/* Pushes the current state to the units that registered since the last push (cheap when there are
 * none).  Library entry points do this on their own; code that loads a code object after
 * nvshmem_init and starts its kernels with a plain launch calls it before the first launch (the
 * reference's nvshmemx_cumodule_init plays this role, src/include/host/nvshmemx_api.h:74). */
NVSHMEMI_HOST_ONLY int nvshmemx_amd_module_init(void);

/* Bounded device waits (counterpart of the reference's NVSHMEM_TIMEOUT_DEVICE_POLLING build,
 * src/include/non_abi/device/wait/nvshmemi_wait_until_apis.cuh:19-35): a wait that polls more than
 * `polls` times records {n, address, found, expected}, n >= 1 being its number among all timeouts of the GPU
 * since nvshmem_init, and returns.  0 = wait forever. */
NVSHMEMI_HOST_ONLY void nvshmemx_amd_set_spin_limit(uint64_t polls);
/* Order of the signal of every device-side put-with-signal whose sig_op does not choose for itself:
 * 0 = the reference's (src/include/non_abi/device/common/nvshmemi_common_device.cuh:529-561: a full fence
 * in front of the signal, here a write-back of the XCD's L2 per call), non-zero = behind the payload of
 * that put only (NVSHMEMX_AMD_SIGNAL_PAYLOAD_ONLY).  The default is 0 unless the environment holds
 * NVSHMEM_AMD_PUT_SIGNAL_ORDER=payload at nvshmem_init.  Waits for the device. */
NVSHMEMI_HOST_ONLY void nvshmemx_amd_set_put_signal_order(int payload_only);
NVSHMEMI_HOST_ONLY int nvshmemx_amd_get_put_signal_order(void); /* 1 = payload only, 0 = the reference's */
/* Copies PE `pe`'s timeout record (4 words) to `out` and clears it; returns its first word (0: none). */
NVSHMEMI_HOST_ONLY uint64_t nvshmemx_amd_read_timeout(int pe, uint64_t out[4]);
/* A wait that gives up does not stay silent.  The device counts every one; the host calls that wait
 * for the device - nvshmem_quiet, nvshmem_fence, nvshmem_barrier_all / nvshmem_sync_all, nvshmem_barrier /
 * nvshmem_team_sync (which then return non-zero), nvshmem_free, nvshmem_finalize - compare the count
 * with what they reported before, and for new timeouts print a message (how many, the spin limit, one
 * PE's record) to stderr and leave it in nvshmemx_amd_last_error().  This call returns the count since
 * nvshmem_init without reporting or clearing anything. */
NVSHMEMI_HOST_ONLY uint64_t nvshmemx_amd_timeout_count(void);

/* Last error text of the calling thread ("" if none); argument errors are reported here and as a
 * non-zero return instead of terminating the process. */
NVSHMEMI_HOST_ONLY const char *nvshmemx_amd_last_error(void);

/* ---- symmetric-space allocator, exposed on its own so it can be exercised without a GPU ----
 * (reference class mspace, src/host/mem/custom_malloc.cpp:74-237).  Addresses are plain integers. */
typedef struct nvshmemi_amd_mspace nvshmemi_amd_mspace_t;
NVSHMEMI_HOST_ONLY nvshmemi_amd_mspace_t *nvshmemi_amd_mspace_create(uint64_t base,
                                                                     uint64_t capacity);
NVSHMEMI_HOST_ONLY void nvshmemi_amd_mspace_destroy(nvshmemi_amd_mspace_t *m);
NVSHMEMI_HOST_ONLY uint64_t nvshmemi_amd_mspace_allocate(nvshmemi_amd_mspace_t *m, uint64_t bytes);
NVSHMEMI_HOST_ONLY uint64_t nvshmemi_amd_mspace_allocate_aligned(nvshmemi_amd_mspace_t *m,
                                                                 uint64_t alignment,
                                                                 uint64_t bytes);
/* Returns 0 on success, -1 if `addr` is not the start of a live allocation. */
NVSHMEMI_HOST_ONLY int nvshmemi_amd_mspace_deallocate(nvshmemi_amd_mspace_t *m, uint64_t addr);
/* Grow/shrink in place when possible; *moved_from is set to the old address when the block moved
 * (the caller copies the payload), else 0.  Returns the new address or 0 when out of space. */
NVSHMEMI_HOST_ONLY uint64_t nvshmemi_amd_mspace_reallocate(nvshmemi_amd_mspace_t *m, uint64_t addr,
                                                           uint64_t bytes, uint64_t *moved_from);
NVSHMEMI_HOST_ONLY uint64_t nvshmemi_amd_mspace_inuse_size(nvshmemi_amd_mspace_t *m,
                                                           uint64_t addr);
NVSHMEMI_HOST_ONLY uint64_t nvshmemi_amd_mspace_free_bytes(nvshmemi_amd_mspace_t *m);
NVSHMEMI_HOST_ONLY uint64_t nvshmemi_amd_mspace_free_chunks(nvshmemi_amd_mspace_t *m);

#ifdef __cplusplus
}
#endif

#endif
