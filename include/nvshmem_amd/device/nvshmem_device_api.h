/*
 * Public device API: the reference's names stamped over the templates of nvshmemi_device.h.
 *   thread scope  nvshmem_*            reference src/include/device/nvshmem_defines.h:80-740
 *   warp / block  nvshmemx_*_{warp,block}  reference src/include/device/nvshmemx_defines.h:35-451
 *   collectives   reference src/include/device/nvshmem_coll_defines.cuh:17-116,
 *                 src/include/device/nvshmemx_coll_defines.cuh:16-175
 * "_warp" means one 64-lane wavefront here.  Device functions share their names with the host
 * entry points; hipcc keeps the two apart by target.
 */
#ifndef NVSHMEM_AMD_DEVICE_API_H
#define NVSHMEM_AMD_DEVICE_API_H

#include "nvshmemi_device.h"

#define NVSHMEMI_DEV static __device__ __forceinline__

/* ---- identity and translation ---- */
NVSHMEMI_DEV int nvshmem_my_pe(void) { return nvshmemi_amd_my_pe(); }
NVSHMEMI_DEV int nvshmem_n_pes(void) { return nvshmemi_amd_n_pes(); }
NVSHMEMI_DEV int nvshmem_team_my_pe(nvshmem_team_t team) { return nvshmemi_team_my_pe(team); }
NVSHMEMI_DEV int nvshmem_team_n_pes(nvshmem_team_t team) { return nvshmemi_team_n_pes(team); }
NVSHMEMI_DEV int nvshmem_team_translate_pe(nvshmem_team_t src_team, int src_pe,
                                           nvshmem_team_t dest_team) {
    return nvshmemi_team_translate_pe(src_team, src_pe, dest_team);
}
NVSHMEMI_DEV void *nvshmem_ptr(const void *ptr, int pe) { return nvshmemi_ptr(ptr, pe); }

/* ---- ordering ---- */
NVSHMEMI_DEV void nvshmem_quiet(void) { nvshmemi_quiet<NVSHMEMI_THREADGROUP_THREAD>(); }
NVSHMEMI_DEV void nvshmem_fence(void) { nvshmemi_quiet<NVSHMEMI_THREADGROUP_THREAD>(); }
NVSHMEMI_DEV void nvshmemx_quiet_warp(void) { nvshmemi_quiet<NVSHMEMI_THREADGROUP_WARP>(); }
NVSHMEMI_DEV void nvshmemx_quiet_block(void) { nvshmemi_quiet<NVSHMEMI_THREADGROUP_BLOCK>(); }

/* ---- barrier / sync over all PEs or a team: one thread group per member PE calls ---- */
#define NVSHMEMI_STAMP_BARRIER(PFX, SFX, SC)                                                     \
    NVSHMEMI_DEV void PFX##_barrier_all##SFX(void) { nvshmemi_barrier_threadgroup<SC>(); }       \
    NVSHMEMI_DEV int PFX##_barrier##SFX(nvshmem_team_t team) {                                   \
        nvshmemi_barrier_threadgroup<SC>(team);                                                  \
        return 0;                                                                                \
    }                                                                                            \
    NVSHMEMI_DEV void PFX##_sync_all##SFX(void) { nvshmemi_sync_threadgroup<SC>(); }             \
    NVSHMEMI_DEV int PFX##_team_sync##SFX(nvshmem_team_t team) {                                 \
        nvshmemi_sync_threadgroup<SC>(team);                                                     \
        return 0;                                                                                \
    }
NVSHMEMI_STAMP_BARRIER(nvshmem, , NVSHMEMI_THREADGROUP_THREAD)
NVSHMEMI_STAMP_BARRIER(nvshmemx, _warp, NVSHMEMI_THREADGROUP_WARP)
NVSHMEMI_STAMP_BARRIER(nvshmemx, _block, NVSHMEMI_THREADGROUP_BLOCK)
#undef NVSHMEMI_STAMP_BARRIER

/* ---- byte RMA ---- */
#define NVSHMEMI_STAMP_MEM_RMA(PFX, SFX, SC)                                                      \
    NVSHMEMI_DEV void PFX##_putmem##SFX(void *dest, const void *source, size_t bytes, int pe) {   \
        nvshmemi_put<char, SC>((char *)dest, (const char *)source, bytes, pe);                    \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_getmem##SFX(void *dest, const void *source, size_t bytes, int pe) {   \
        nvshmemi_get<char, SC>((char *)dest, (const char *)source, bytes, pe);                    \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_putmem_nbi##SFX(void *dest, const void *source, size_t bytes,         \
                                            int pe) {                                             \
        nvshmemi_put<char, SC>((char *)dest, (const char *)source, bytes, pe);                    \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_getmem_nbi##SFX(void *dest, const void *source, size_t bytes,         \
                                            int pe) {                                             \
        nvshmemi_get<char, SC>((char *)dest, (const char *)source, bytes, pe);                    \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_putmem_signal##SFX(void *dest, const void *source, size_t bytes,      \
                                               uint64_t *sig_addr, uint64_t signal, int sig_op,   \
                                               int pe) {                                          \
        nvshmemi_put_signal<char, SC>((char *)dest, (const char *)source, bytes, sig_addr,        \
                                      signal, sig_op, pe);                                        \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_putmem_signal_nbi##SFX(void *dest, const void *source, size_t bytes,  \
                                                   uint64_t *sig_addr, uint64_t signal,           \
                                                   int sig_op, int pe) {                          \
        nvshmemi_put_signal<char, SC>((char *)dest, (const char *)source, bytes, sig_addr,        \
                                      signal, sig_op, pe);                                        \
    }
NVSHMEMI_STAMP_MEM_RMA(nvshmem, , NVSHMEMI_THREADGROUP_THREAD)
NVSHMEMI_STAMP_MEM_RMA(nvshmemx, _warp, NVSHMEMI_THREADGROUP_WARP)
NVSHMEMI_STAMP_MEM_RMA(nvshmemx, _block, NVSHMEMI_THREADGROUP_BLOCK)
#undef NVSHMEMI_STAMP_MEM_RMA

/* ---- typed RMA: 25 types x 3 scopes ---- */
#define NVSHMEMI_STAMP_TYPED_RMA_SCOPE(NAME, TYPE, PFX, SFX, SC)                                  \
    NVSHMEMI_DEV void PFX##_##NAME##_put##SFX(TYPE *dest, const TYPE *source, size_t nelems,      \
                                              int pe) {                                           \
        nvshmemi_put<TYPE, SC>(dest, source, nelems, pe);                                         \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_##NAME##_get##SFX(TYPE *dest, const TYPE *source, size_t nelems,      \
                                              int pe) {                                           \
        nvshmemi_get<TYPE, SC>(dest, source, nelems, pe);                                         \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_##NAME##_put_nbi##SFX(TYPE *dest, const TYPE *source, size_t nelems,  \
                                                  int pe) {                                       \
        nvshmemi_put<TYPE, SC>(dest, source, nelems, pe);                                         \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_##NAME##_get_nbi##SFX(TYPE *dest, const TYPE *source, size_t nelems,  \
                                                  int pe) {                                       \
        nvshmemi_get<TYPE, SC>(dest, source, nelems, pe);                                         \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_##NAME##_iput##SFX(TYPE *dest, const TYPE *source, ptrdiff_t dst,     \
                                               ptrdiff_t sst, size_t nelems, int pe) {            \
        nvshmemi_iput<TYPE, SC>(dest, source, dst, sst, nelems, pe);                              \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_##NAME##_iget##SFX(TYPE *dest, const TYPE *source, ptrdiff_t dst,     \
                                               ptrdiff_t sst, size_t nelems, int pe) {            \
        nvshmemi_iget<TYPE, SC>(dest, source, dst, sst, nelems, pe);                              \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_##NAME##_put_signal##SFX(TYPE *dest, const TYPE *source,              \
                                                     size_t nelems, uint64_t *sig_addr,           \
                                                     uint64_t signal, int sig_op, int pe) {       \
        nvshmemi_put_signal<TYPE, SC>(dest, source, nelems, sig_addr, signal, sig_op, pe);        \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_##NAME##_put_signal_nbi##SFX(TYPE *dest, const TYPE *source,          \
                                                         size_t nelems, uint64_t *sig_addr,       \
                                                         uint64_t signal, int sig_op, int pe) {   \
        nvshmemi_put_signal<TYPE, SC>(dest, source, nelems, sig_addr, signal, sig_op, pe);        \
    }
#define NVSHMEMI_STAMP_TYPED_RMA(NAME, TYPE, TAG)                                                 \
    NVSHMEMI_DEV void nvshmem_##NAME##_p(TYPE *dest, const TYPE value, int pe) {                  \
        nvshmemi_p<TYPE>(dest, value, pe);                                                        \
    }                                                                                             \
    NVSHMEMI_DEV TYPE nvshmem_##NAME##_g(const TYPE *source, int pe) {                            \
        return nvshmemi_g<TYPE>(source, pe);                                                      \
    }                                                                                             \
    NVSHMEMI_STAMP_TYPED_RMA_SCOPE(NAME, TYPE, nvshmem, , NVSHMEMI_THREADGROUP_THREAD)            \
    NVSHMEMI_STAMP_TYPED_RMA_SCOPE(NAME, TYPE, nvshmemx, _warp, NVSHMEMI_THREADGROUP_WARP)        \
    NVSHMEMI_STAMP_TYPED_RMA_SCOPE(NAME, TYPE, nvshmemx, _block, NVSHMEMI_THREADGROUP_BLOCK)
NVSHMEMI_REPT_FOR_STANDARD_RMA_TYPES(NVSHMEMI_STAMP_TYPED_RMA)
#undef NVSHMEMI_STAMP_TYPED_RMA
#undef NVSHMEMI_STAMP_TYPED_RMA_SCOPE

/* ---- sized RMA put8..put128: nelems elements of BITS/8 bytes ---- */
template <int BYTES> struct nvshmemi_amd_sized;
template <> struct nvshmemi_amd_sized<1> { typedef uint8_t type; };
template <> struct nvshmemi_amd_sized<2> { typedef uint16_t type; };
template <> struct nvshmemi_amd_sized<4> { typedef uint32_t type; };
template <> struct nvshmemi_amd_sized<8> { typedef uint64_t type; };
template <> struct nvshmemi_amd_sized<16> { typedef nvshmemi_v4u type; };
#define NVSHMEMI_STAMP_SIZED_RMA_SCOPE(BITS, BYTES, PFX, SFX, SC)                                 \
    NVSHMEMI_DEV void PFX##_put##BITS##SFX(void *dest, const void *source, size_t nelems,         \
                                           int pe) {                                              \
        nvshmemi_put<char, SC>((char *)dest, (const char *)source, nelems * BYTES, pe);           \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_get##BITS##SFX(void *dest, const void *source, size_t nelems,         \
                                           int pe) {                                              \
        nvshmemi_get<char, SC>((char *)dest, (const char *)source, nelems * BYTES, pe);           \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_put##BITS##_nbi##SFX(void *dest, const void *source, size_t nelems,   \
                                                 int pe) {                                        \
        nvshmemi_put<char, SC>((char *)dest, (const char *)source, nelems * BYTES, pe);           \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_get##BITS##_nbi##SFX(void *dest, const void *source, size_t nelems,   \
                                                 int pe) {                                        \
        nvshmemi_get<char, SC>((char *)dest, (const char *)source, nelems * BYTES, pe);           \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_iput##BITS##SFX(void *dest, const void *source, ptrdiff_t dst,        \
                                            ptrdiff_t sst, size_t nelems, int pe) {               \
        nvshmemi_iput<nvshmemi_amd_sized<BYTES>::type, SC>(                                       \
            (nvshmemi_amd_sized<BYTES>::type *)dest,                                              \
            (const nvshmemi_amd_sized<BYTES>::type *)source, dst, sst, nelems, pe);               \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_iget##BITS##SFX(void *dest, const void *source, ptrdiff_t dst,        \
                                            ptrdiff_t sst, size_t nelems, int pe) {               \
        nvshmemi_iget<nvshmemi_amd_sized<BYTES>::type, SC>(                                       \
            (nvshmemi_amd_sized<BYTES>::type *)dest,                                              \
            (const nvshmemi_amd_sized<BYTES>::type *)source, dst, sst, nelems, pe);               \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_put##BITS##_signal##SFX(void *dest, const void *source,               \
                                                    size_t nelems, uint64_t *sig_addr,            \
                                                    uint64_t signal, int sig_op, int pe) {        \
        nvshmemi_put_signal<char, SC>((char *)dest, (const char *)source, nelems * BYTES,         \
                                      sig_addr, signal, sig_op, pe);                              \
    }                                                                                             \
    NVSHMEMI_DEV void PFX##_put##BITS##_signal_nbi##SFX(void *dest, const void *source,           \
                                                        size_t nelems, uint64_t *sig_addr,        \
                                                        uint64_t signal, int sig_op, int pe) {    \
        nvshmemi_put_signal<char, SC>((char *)dest, (const char *)source, nelems * BYTES,         \
                                      sig_addr, signal, sig_op, pe);                              \
    }
#define NVSHMEMI_STAMP_SIZED_RMA(BITS, BYTES)                                                     \
    NVSHMEMI_STAMP_SIZED_RMA_SCOPE(BITS, BYTES, nvshmem, , NVSHMEMI_THREADGROUP_THREAD)           \
    NVSHMEMI_STAMP_SIZED_RMA_SCOPE(BITS, BYTES, nvshmemx, _warp, NVSHMEMI_THREADGROUP_WARP)       \
    NVSHMEMI_STAMP_SIZED_RMA_SCOPE(BITS, BYTES, nvshmemx, _block, NVSHMEMI_THREADGROUP_BLOCK)
NVSHMEMI_REPT_FOR_SIZES(NVSHMEMI_STAMP_SIZED_RMA)
#undef NVSHMEMI_STAMP_SIZED_RMA
#undef NVSHMEMI_STAMP_SIZED_RMA_SCOPE

/* ---- signals ---- */
/* As in the reference (nvshmemi_signal_op, common/nvshmemi_common_device.cuh:507-527: a bare store or
 * atomic add), a standalone signal orders nothing by itself: a caller that publishes data with it
 * calls nvshmem_fence or nvshmem_quiet first, or uses a put-with-signal. */
NVSHMEMI_DEV void nvshmemx_signal_op(uint64_t *sig_addr, uint64_t signal, int sig_op, int pe) {
    nvshmemi_signal_op(sig_addr, signal, sig_op, pe);
}
NVSHMEMI_DEV uint64_t nvshmem_signal_fetch(uint64_t *sig_addr) {
    return nvshmemi_amd_poll(reinterpret_cast<const uint64_t *>(nvshmemi_amd_local(sig_addr)));
}
NVSHMEMI_DEV uint64_t nvshmem_signal_wait_until(uint64_t *sig_addr, int cmp, uint64_t cmp_val) {
    return nvshmemi_wait_until<uint64_t>(sig_addr, cmp, cmp_val);
}

/* ---- typed wait / test (14 types): scalar, all / any / some, and the _vector forms ---- */
#define NVSHMEMI_STAMP_WAIT(NAME, TYPE)                                                           \
    NVSHMEMI_DEV void nvshmem_##NAME##_wait_until(TYPE *ivar, int cmp, TYPE cmp_value) {          \
        nvshmemi_wait_until<TYPE>(ivar, cmp, cmp_value);                                          \
    }                                                                                             \
    NVSHMEMI_DEV int nvshmem_##NAME##_test(TYPE *ivar, int cmp, TYPE cmp_value) {                 \
        return nvshmemi_test<TYPE>(ivar, cmp, cmp_value);                                         \
    }                                                                                             \
    NVSHMEMI_DEV void nvshmem_##NAME##_wait_until_all(TYPE *ivars, size_t nelems,                 \
                                                      const int *status, int cmp,                 \
                                                      TYPE cmp_value) {                           \
        nvshmemi_wait_until_all<TYPE, false>(ivars, nelems, status, cmp, &cmp_value);             \
    }                                                                                             \
    NVSHMEMI_DEV size_t nvshmem_##NAME##_wait_until_any(TYPE *ivars, size_t nelems,               \
                                                        const int *status, int cmp,               \
                                                        TYPE cmp_value) {                         \
        return nvshmemi_wait_until_any<TYPE, false>(ivars, nelems, status, cmp, &cmp_value);      \
    }                                                                                             \
    NVSHMEMI_DEV size_t nvshmem_##NAME##_wait_until_some(TYPE *ivars, size_t nelems,              \
                                                         size_t *indices, const int *status,      \
                                                         int cmp, TYPE cmp_value) {               \
        return nvshmemi_wait_until_some<TYPE, false>(ivars, nelems, indices, status, cmp,         \
                                                     &cmp_value);                                 \
    }                                                                                             \
    NVSHMEMI_DEV void nvshmem_##NAME##_wait_until_all_vector(TYPE *ivars, size_t nelems,          \
                                                             const int *status, int cmp,          \
                                                             TYPE *cmp_values) {                  \
        nvshmemi_wait_until_all<TYPE, true>(ivars, nelems, status, cmp, cmp_values);              \
    }                                                                                             \
    NVSHMEMI_DEV size_t nvshmem_##NAME##_wait_until_any_vector(TYPE *ivars, size_t nelems,        \
                                                               const int *status, int cmp,        \
                                                               TYPE *cmp_values) {                \
        return nvshmemi_wait_until_any<TYPE, true>(ivars, nelems, status, cmp, cmp_values);       \
    }                                                                                             \
    NVSHMEMI_DEV size_t nvshmem_##NAME##_wait_until_some_vector(TYPE *ivars, size_t nelems,       \
                                                                size_t *indices,                  \
                                                                const int *status, int cmp,       \
                                                                TYPE *cmp_values) {               \
        return nvshmemi_wait_until_some<TYPE, true>(ivars, nelems, indices, status, cmp,          \
                                                    cmp_values);                                  \
    }                                                                                             \
    NVSHMEMI_DEV int nvshmem_##NAME##_test_all(TYPE *ivars, size_t nelems, const int *status,     \
                                               int cmp, TYPE cmp_value) {                         \
        return nvshmemi_test_all<TYPE, false>(ivars, nelems, status, cmp, &cmp_value);            \
    }                                                                                             \
    NVSHMEMI_DEV size_t nvshmem_##NAME##_test_any(TYPE *ivars, size_t nelems, const int *status,  \
                                                  int cmp, TYPE cmp_value) {                      \
        return nvshmemi_test_any<TYPE, false>(ivars, nelems, status, cmp, &cmp_value);            \
    }                                                                                             \
    NVSHMEMI_DEV size_t nvshmem_##NAME##_test_some(TYPE *ivars, size_t nelems, size_t *indices,   \
                                                   const int *status, int cmp, TYPE cmp_value) {  \
        return nvshmemi_test_some<TYPE, false>(ivars, nelems, indices, status, cmp, &cmp_value);  \
    }                                                                                             \
    NVSHMEMI_DEV int nvshmem_##NAME##_test_all_vector(TYPE *ivars, size_t nelems,                 \
                                                      const int *status, int cmp,                 \
                                                      TYPE *cmp_values) {                         \
        return nvshmemi_test_all<TYPE, true>(ivars, nelems, status, cmp, cmp_values);             \
    }                                                                                             \
    NVSHMEMI_DEV size_t nvshmem_##NAME##_test_any_vector(TYPE *ivars, size_t nelems,              \
                                                         const int *status, int cmp,              \
                                                         TYPE *cmp_values) {                      \
        return nvshmemi_test_any<TYPE, true>(ivars, nelems, status, cmp, cmp_values);             \
    }                                                                                             \
    NVSHMEMI_DEV size_t nvshmem_##NAME##_test_some_vector(TYPE *ivars, size_t nelems,             \
                                                          size_t *indices, const int *status,     \
                                                          int cmp, TYPE *cmp_values) {            \
        return nvshmemi_test_some<TYPE, true>(ivars, nelems, indices, status, cmp, cmp_values);   \
    }
NVSHMEMI_REPT_FOR_WAIT_TYPES(NVSHMEMI_STAMP_WAIT)
#undef NVSHMEMI_STAMP_WAIT

/* ---- atomic memory operations (reference nvshmem_defines.h:742-1236) ---- */
#define NVSHMEMI_STAMP_AMO_FETCH_SET_SWAP(NAME, TYPE)                                             \
    NVSHMEMI_DEV TYPE nvshmem_##NAME##_atomic_fetch(const TYPE *target, int pe) {                 \
        return nvshmemi_atomic_fetch<TYPE>(target, pe);                                           \
    }                                                                                             \
    NVSHMEMI_DEV void nvshmem_##NAME##_atomic_set(TYPE *target, TYPE value, int pe) {             \
        nvshmemi_atomic_set<TYPE>(target, value, pe);                                             \
    }                                                                                             \
    NVSHMEMI_DEV TYPE nvshmem_##NAME##_atomic_swap(TYPE *target, TYPE value, int pe) {            \
        return nvshmemi_atomic_swap<TYPE>(target, value, pe);                                     \
    }
NVSHMEMI_REPT_FOR_STANDARD_AMO_TYPES(NVSHMEMI_STAMP_AMO_FETCH_SET_SWAP)
NVSHMEMI_REPT_FOR_EXTENDED_AMO_TYPES(NVSHMEMI_STAMP_AMO_FETCH_SET_SWAP)
#undef NVSHMEMI_STAMP_AMO_FETCH_SET_SWAP

#define NVSHMEMI_STAMP_AMO_ARITH(NAME, TYPE)                                                      \
    NVSHMEMI_DEV TYPE nvshmem_##NAME##_atomic_compare_swap(TYPE *target, TYPE cond, TYPE value,   \
                                                           int pe) {                              \
        return nvshmemi_atomic_compare_swap<TYPE>(target, cond, value, pe);                       \
    }                                                                                             \
    NVSHMEMI_DEV TYPE nvshmem_##NAME##_atomic_fetch_add(TYPE *target, TYPE value, int pe) {       \
        return nvshmemi_atomic_fetch_add<TYPE>(target, value, pe);                                \
    }                                                                                             \
    NVSHMEMI_DEV void nvshmem_##NAME##_atomic_add(TYPE *target, TYPE value, int pe) {             \
        (void)nvshmemi_atomic_fetch_add<TYPE>(target, value, pe);                                 \
    }                                                                                             \
    NVSHMEMI_DEV TYPE nvshmem_##NAME##_atomic_fetch_inc(TYPE *target, int pe) {                   \
        return nvshmemi_atomic_fetch_add<TYPE>(target, (TYPE)1, pe);                              \
    }                                                                                             \
    NVSHMEMI_DEV void nvshmem_##NAME##_atomic_inc(TYPE *target, int pe) {                         \
        (void)nvshmemi_atomic_fetch_add<TYPE>(target, (TYPE)1, pe);                               \
    }
NVSHMEMI_REPT_FOR_STANDARD_AMO_TYPES(NVSHMEMI_STAMP_AMO_ARITH)
#undef NVSHMEMI_STAMP_AMO_ARITH

#define NVSHMEMI_STAMP_AMO_BITWISE(NAME, TYPE)                                                    \
    NVSHMEMI_DEV TYPE nvshmem_##NAME##_atomic_fetch_and(TYPE *target, TYPE value, int pe) {       \
        return nvshmemi_atomic_fetch_and<TYPE>(target, value, pe);                                \
    }                                                                                             \
    NVSHMEMI_DEV TYPE nvshmem_##NAME##_atomic_fetch_or(TYPE *target, TYPE value, int pe) {        \
        return nvshmemi_atomic_fetch_or<TYPE>(target, value, pe);                                 \
    }                                                                                             \
    NVSHMEMI_DEV TYPE nvshmem_##NAME##_atomic_fetch_xor(TYPE *target, TYPE value, int pe) {       \
        return nvshmemi_atomic_fetch_xor<TYPE>(target, value, pe);                                \
    }                                                                                             \
    NVSHMEMI_DEV void nvshmem_##NAME##_atomic_and(TYPE *target, TYPE value, int pe) {             \
        (void)nvshmemi_atomic_fetch_and<TYPE>(target, value, pe);                                 \
    }                                                                                             \
    NVSHMEMI_DEV void nvshmem_##NAME##_atomic_or(TYPE *target, TYPE value, int pe) {              \
        (void)nvshmemi_atomic_fetch_or<TYPE>(target, value, pe);                                  \
    }                                                                                             \
    NVSHMEMI_DEV void nvshmem_##NAME##_atomic_xor(TYPE *target, TYPE value, int pe) {             \
        (void)nvshmemi_atomic_fetch_xor<TYPE>(target, value, pe);                                 \
    }
NVSHMEMI_REPT_FOR_BITWISE_AMO_TYPES(NVSHMEMI_STAMP_AMO_BITWISE)
#undef NVSHMEMI_STAMP_AMO_BITWISE

/* ---- collectives inside a kernel: one thread group per PE ---- */
#define NVSHMEMI_STAMP_COLL_SCOPE(NAME, TYPE, PFX, SFX, SC)                                       \
    NVSHMEMI_DEV int PFX##_##NAME##_alltoall##SFX(nvshmem_team_t team, TYPE *dest,                \
                                                  const TYPE *src, size_t nelems) {               \
        return nvshmemi_alltoall_threadgroup<TYPE, SC>(team, dest, src, nelems);                  \
    }                                                                                             \
    NVSHMEMI_DEV int PFX##_##NAME##_fcollect##SFX(nvshmem_team_t team, TYPE *dest,                \
                                                  const TYPE *src, size_t nelems) {               \
        return nvshmemi_fcollect_threadgroup<TYPE, SC>(team, dest, src, nelems);                  \
    }                                                                                             \
    NVSHMEMI_DEV int PFX##_##NAME##_broadcast##SFX(nvshmem_team_t team, TYPE *dest,               \
                                                   const TYPE *src, size_t nelems, int PE_root) { \
        return nvshmemi_broadcast_threadgroup<TYPE, SC>(team, dest, src, nelems, PE_root);        \
    }
#define NVSHMEMI_STAMP_COLL(NAME, TYPE, TAG)                                                      \
    NVSHMEMI_STAMP_COLL_SCOPE(NAME, TYPE, nvshmem, , NVSHMEMI_THREADGROUP_THREAD)                 \
    NVSHMEMI_STAMP_COLL_SCOPE(NAME, TYPE, nvshmemx, _warp, NVSHMEMI_THREADGROUP_WARP)             \
    NVSHMEMI_STAMP_COLL_SCOPE(NAME, TYPE, nvshmemx, _block, NVSHMEMI_THREADGROUP_BLOCK)
NVSHMEMI_REPT_FOR_STANDARD_RMA_TYPES(NVSHMEMI_STAMP_COLL)
#undef NVSHMEMI_STAMP_COLL
#undef NVSHMEMI_STAMP_COLL_SCOPE

#define NVSHMEMI_STAMP_MEM_COLL(PFX, SFX, SC)                                                     \
    NVSHMEMI_DEV int PFX##_alltoallmem##SFX(nvshmem_team_t team, void *dest, const void *src,     \
                                            size_t nelems) {                                      \
        return nvshmemi_alltoall_threadgroup<char, SC>(team, (char *)dest, (const char *)src,     \
                                                       nelems);                                   \
    }                                                                                             \
    NVSHMEMI_DEV int PFX##_fcollectmem##SFX(nvshmem_team_t team, void *dest, const void *src,     \
                                            size_t nelems) {                                      \
        return nvshmemi_fcollect_threadgroup<char, SC>(team, (char *)dest, (const char *)src,     \
                                                       nelems);                                   \
    }                                                                                             \
    NVSHMEMI_DEV int PFX##_broadcastmem##SFX(nvshmem_team_t team, void *dest, const void *src,    \
                                             size_t nelems, int PE_root) {                        \
        return nvshmemi_broadcast_threadgroup<char, SC>(team, (char *)dest, (const char *)src,    \
                                                        nelems, PE_root);                         \
    }
NVSHMEMI_STAMP_MEM_COLL(nvshmem, , NVSHMEMI_THREADGROUP_THREAD)
NVSHMEMI_STAMP_MEM_COLL(nvshmemx, _warp, NVSHMEMI_THREADGROUP_WARP)
NVSHMEMI_STAMP_MEM_COLL(nvshmemx, _block, NVSHMEMI_THREADGROUP_BLOCK)
#undef NVSHMEMI_STAMP_MEM_COLL

#define NVSHMEMI_STAMP_REDUCE(NAME, TYPE, TAG, OP)                                                \
    NVSHMEMI_DEV int nvshmem_##NAME##_##OP##_reduce(nvshmem_team_t team, TYPE *dest,              \
                                                    const TYPE *src, size_t nreduce) {            \
        return nvshmemi_reduce_threadgroup<TYPE, NVSHMEMI_OP_##OP, NVSHMEMI_THREADGROUP_THREAD>(  \
            team, dest, src, nreduce);                                                            \
    }                                                                                             \
    NVSHMEMI_DEV int nvshmemx_##NAME##_##OP##_reduce_warp(nvshmem_team_t team, TYPE *dest,        \
                                                          const TYPE *src, size_t nreduce) {      \
        return nvshmemi_reduce_threadgroup<TYPE, NVSHMEMI_OP_##OP, NVSHMEMI_THREADGROUP_WARP>(    \
            team, dest, src, nreduce);                                                            \
    }                                                                                             \
    NVSHMEMI_DEV int nvshmemx_##NAME##_##OP##_reduce_block(nvshmem_team_t team, TYPE *dest,       \
                                                           const TYPE *src, size_t nreduce) {     \
        return nvshmemi_reduce_threadgroup<TYPE, NVSHMEMI_OP_##OP, NVSHMEMI_THREADGROUP_BLOCK>(   \
            team, dest, src, nreduce);                                                            \
    }                                                                                             \
    NVSHMEMI_DEV int nvshmem_##NAME##_##OP##_reducescatter(nvshmem_team_t team, TYPE *dest,       \
                                                           const TYPE *src, size_t nreduce) {     \
        return nvshmemi_reducescatter_threadgroup<TYPE, NVSHMEMI_OP_##OP,                         \
                                                  NVSHMEMI_THREADGROUP_THREAD>(team, dest, src,   \
                                                                               nreduce);          \
    }                                                                                             \
    NVSHMEMI_DEV int nvshmemx_##NAME##_##OP##_reducescatter_warp(nvshmem_team_t team, TYPE *dest, \
                                                                 const TYPE *src,                 \
                                                                 size_t nreduce) {                \
        return nvshmemi_reducescatter_threadgroup<TYPE, NVSHMEMI_OP_##OP,                         \
                                                  NVSHMEMI_THREADGROUP_WARP>(team, dest, src,     \
                                                                             nreduce);            \
    }                                                                                             \
    NVSHMEMI_DEV int nvshmemx_##NAME##_##OP##_reducescatter_block(nvshmem_team_t team,            \
                                                                  TYPE *dest, const TYPE *src,    \
                                                                  size_t nreduce) {               \
        return nvshmemi_reducescatter_threadgroup<TYPE, NVSHMEMI_OP_##OP,                         \
                                                  NVSHMEMI_THREADGROUP_BLOCK>(team, dest, src,    \
                                                                              nreduce);           \
    }
NVSHMEMI_REPT_FOR_ALL_REDUCE_TYPES_AND_OPS(NVSHMEMI_STAMP_REDUCE)
#undef NVSHMEMI_STAMP_REDUCE

/* barrier among the PEs of `team`, called by one warpgroup (256 threads: four wavefronts) per PE
 * (reference nvshmemx_coll_api.h:118, nvshmemx_coll_defines.cuh:52) */
NVSHMEMI_DEV int nvshmemx_barrier_warpgroup(nvshmem_team_t team) { return nvshmemi_barrier_warpgroup(team); }

/* (value, location) maximum, block scope only (reference nvshmemx_coll_defines.cuh:210-214) */
NVSHMEMI_DEV int nvshmemx_double2_maxloc_reduce_block(nvshmem_team_t team, double2 *dest,
                                                      const double2 *source, size_t nreduce) {
    return nvshmemi_double2_maxloc_reduce_block(team, dest, source, nreduce);
}

/* ---- library identification from device code (reference nvshmem_defines.h:63-77) ---- */
NVSHMEMI_DEV void nvshmem_info_get_version(int *major, int *minor) {
    if (major) *major = NVSHMEM_MAJOR_VERSION;
    if (minor) *minor = NVSHMEM_MINOR_VERSION;
}
/* name receives at most NVSHMEM_MAX_NAME_LEN bytes including the terminator */
NVSHMEMI_DEV void nvshmem_info_get_name(char *name) {
    static constexpr char vendor[] = NVSHMEM_VENDOR_STRING;
    constexpr size_t len = sizeof(vendor) < NVSHMEM_MAX_NAME_LEN ? sizeof(vendor) : NVSHMEM_MAX_NAME_LEN;
    if (!name) return;
    for (size_t k = 0; k + 1 < len; ++k) name[k] = vendor[k];
    name[len - 1] = 0;
}
NVSHMEMI_DEV void nvshmemx_vendor_get_version_info(int *major, int *minor, int *patch) {
    if (major) *major = NVSHMEM_VENDOR_MAJOR_VERSION;
    if (minor) *minor = NVSHMEM_VENDOR_MINOR_VERSION;
    if (patch) *patch = NVSHMEM_VENDOR_PATCH_VERSION;
}

#undef NVSHMEMI_DEV
#endif
