// Atomic memory operations through the public device API: one kernel that applies every stamped
// (type, operation) pair once to a slot nobody else touches, so the outcome is predictable on the
// host, and one in which all threads of all PEs contend for the same words.  The operation families
// are those of the reference's src/include/device/nvshmem_defines.h:742-1236 (which its
// perftest/device/pt-to-pt/shmem_atomic_*.cu files time without checking values).
#include <hip/hip_runtime.h>

#include "nvshmem_perftest.h"
#include "nvshmemx.h"
#include "perftest_common.hpp"

namespace {

template <typename T>
__device__ void record(uint64_t *out, int k, T fetched) {
    uint64_t w = 0;
    __builtin_memcpy(&w, &fetched, sizeof fetched);
    out[k] = w;
}
template <typename T>
__device__ T operand(const uint64_t *words, int k) {
    T v;
    __builtin_memcpy(&v, &words[k], sizeof v);
    return v;
}

// slots, val, cond, out: symmetric arrays of 64-bit words, one word per case.  Case k acts on the
// low sizeof(TYPE) bytes of slots[k] on the right neighbour with the operands val[k] (and cond[k]
// for compare_swap) read from the caller's own copies, and stores what the call returned into the
// caller's out[k].  Case order: fetch, set, swap for the standard then the extended types;
// compare_swap (twice: cond[k] and cond[k+1]), fetch_add, add, fetch_inc, inc for the standard
// types; fetch_and, and, fetch_or, or, fetch_xor, xor for the bitwise types.
__global__ void amo_matrix_kernel(uint64_t *slots, const uint64_t *val, const uint64_t *cond,
                                  uint64_t *out, int *ncases) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const int me = nvshmem_my_pe(), peer = (me + 1) % nvshmem_n_pes();
    const uint64_t *v = (const uint64_t *)nvshmem_ptr(val, me);
    const uint64_t *c = (const uint64_t *)nvshmem_ptr(cond, me);
    uint64_t *o = (uint64_t *)nvshmem_ptr(out, me);
    int k = 0;
#define CASES_FETCH_SET_SWAP(NAME, TYPE)                                                          \
    record<TYPE>(o, k, nvshmem_##NAME##_atomic_fetch((const TYPE *)(slots + k), peer)); ++k;      \
    nvshmem_##NAME##_atomic_set((TYPE *)(slots + k), operand<TYPE>(v, k), peer); ++k;             \
    record<TYPE>(o, k, nvshmem_##NAME##_atomic_swap((TYPE *)(slots + k), operand<TYPE>(v, k), peer)); ++k;
    NVSHMEMI_REPT_FOR_STANDARD_AMO_TYPES(CASES_FETCH_SET_SWAP)
    NVSHMEMI_REPT_FOR_EXTENDED_AMO_TYPES(CASES_FETCH_SET_SWAP)
#undef CASES_FETCH_SET_SWAP
#define CASES_ARITH(NAME, TYPE)                                                                   \
    record<TYPE>(o, k, nvshmem_##NAME##_atomic_compare_swap((TYPE *)(slots + k), operand<TYPE>(c, k), \
                                                            operand<TYPE>(v, k), peer)); ++k;     \
    record<TYPE>(o, k, nvshmem_##NAME##_atomic_compare_swap((TYPE *)(slots + k), operand<TYPE>(c, k), \
                                                            operand<TYPE>(v, k), peer)); ++k;     \
    record<TYPE>(o, k, nvshmem_##NAME##_atomic_fetch_add((TYPE *)(slots + k), operand<TYPE>(v, k), peer)); ++k; \
    nvshmem_##NAME##_atomic_add((TYPE *)(slots + k), operand<TYPE>(v, k), peer); ++k;             \
    record<TYPE>(o, k, nvshmem_##NAME##_atomic_fetch_inc((TYPE *)(slots + k), peer)); ++k;        \
    nvshmem_##NAME##_atomic_inc((TYPE *)(slots + k), peer); ++k;
    NVSHMEMI_REPT_FOR_STANDARD_AMO_TYPES(CASES_ARITH)
#undef CASES_ARITH
#define CASES_BITWISE(NAME, TYPE)                                                                 \
    record<TYPE>(o, k, nvshmem_##NAME##_atomic_fetch_and((TYPE *)(slots + k), operand<TYPE>(v, k), peer)); ++k; \
    nvshmem_##NAME##_atomic_and((TYPE *)(slots + k), operand<TYPE>(v, k), peer); ++k;             \
    record<TYPE>(o, k, nvshmem_##NAME##_atomic_fetch_or((TYPE *)(slots + k), operand<TYPE>(v, k), peer)); ++k; \
    nvshmem_##NAME##_atomic_or((TYPE *)(slots + k), operand<TYPE>(v, k), peer); ++k;              \
    record<TYPE>(o, k, nvshmem_##NAME##_atomic_fetch_xor((TYPE *)(slots + k), operand<TYPE>(v, k), peer)); ++k; \
    nvshmem_##NAME##_atomic_xor((TYPE *)(slots + k), operand<TYPE>(v, k), peer); ++k;
    NVSHMEMI_REPT_FOR_BITWISE_AMO_TYPES(CASES_BITWISE)
#undef CASES_BITWISE
    *(int *)nvshmem_ptr(ncases, me) = k;
}

#define COUNT_ONE(NAME, TYPE) +1
constexpr int kStandard = 0 NVSHMEMI_REPT_FOR_STANDARD_AMO_TYPES(COUNT_ONE);
constexpr int kExtended = 0 NVSHMEMI_REPT_FOR_EXTENDED_AMO_TYPES(COUNT_ONE);
constexpr int kBitwise = 0 NVSHMEMI_REPT_FOR_BITWISE_AMO_TYPES(COUNT_ONE);
#undef COUNT_ONE
constexpr int kMatrixCases = 3 * (kStandard + kExtended) + 6 * kStandard + 6 * kBitwise;

// Every thread of every PE, all on PE `home`'s copies:
//   ticket = fetch_add(counter, 1); inc(seen + ticket)   -> seen[0 .. total) all 1, counter == total
//   compare_swap(lock, 0, id + 1)                         -> exactly one thread finds 0
//   xor(bits, 1 << (id % 64)), or(mask, 1 << (id % 64)), and(clear, ~(1 << (id % 64)))
//   fetch_add(fsum32, id) on a 32-bit word, swap(last, id + 1) whose returned values chain
// words: counter, lock, bits, mask, clear, sum32, last, winners (8 uint64); seen: `total` uint32;
// chain: `total` uint64, thread id's entry on PE `home` receives what its swap returned.
__global__ void amo_contend_kernel(uint64_t *words, unsigned int *seen, unsigned long long *chain,
                                   int home) {
    const unsigned long long per_pe = (unsigned long long)gridDim.x * blockDim.x;
    const unsigned long long id =
        (unsigned long long)nvshmem_my_pe() * per_pe + (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
    unsigned long long *w = (unsigned long long *)words;
    const unsigned long long ticket = nvshmem_ulonglong_atomic_fetch_add(w + 0, 1ull, home);
    nvshmem_uint_atomic_inc(seen + ticket, home);
    if (nvshmem_uint64_atomic_compare_swap(words + 1, 0, id + 1, home) == 0)
        nvshmem_int64_atomic_inc((int64_t *)(words + 7), home);
    const uint64_t bit = 1ull << (id % 64);
    nvshmem_uint64_atomic_xor(words + 2, bit, home);
    nvshmem_ulong_atomic_or((unsigned long *)(words + 3), bit, home);
    nvshmem_int64_atomic_and((int64_t *)(words + 4), (int64_t)~bit, home);
    nvshmem_int32_atomic_add((int32_t *)(words + 5), (int32_t)id, home);
    // the values returned by the swaps form a chain that visits every id once
    ((unsigned long long *)nvshmem_ptr(chain, home))[id] = nvshmem_ulonglong_atomic_swap(w + 6, id + 1, home);
}

}  // namespace

extern "C" {

int nvshmem_perftest_amo_matrix_cases(void) { return kMatrixCases; }

int nvshmem_perftest_amo_matrix(uint64_t *slots, const uint64_t *val, const uint64_t *cond,
                                uint64_t *out, int *ncases, void *stream) {
    const size_t bytes = sizeof(uint64_t) * (kMatrixCases + 1);
    if (!perftest::ready() || !perftest::check_range(slots, bytes) ||
        !perftest::check_range(val, bytes) || !perftest::check_range(cond, bytes) ||
        !perftest::check_range(out, bytes) || !perftest::check_range(ncases, sizeof(int)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    hipLaunchKernelGGL(amo_matrix_kernel, dim3(1, 1, (unsigned)nvshmem_n_pes()), dim3(64), 0,
                       (hipStream_t)stream, slots, val, cond, out, ncases);
    return perftest::launch_status("amo_matrix");
}

int nvshmem_perftest_amo_contend(uint64_t *words, unsigned int *seen, unsigned long long *chain,
                                 int home, int blocks, int threads, void *stream) {
    if (!perftest::ready() || !perftest::check_launch(blocks, threads) || home < 0 ||
        home >= nvshmem_n_pes())
        return NVSHMEMX_ERROR_INVALID_VALUE;
    const size_t total = (size_t)blocks * threads * (size_t)nvshmem_n_pes();
    if (!perftest::check_range(words, 8 * sizeof(uint64_t)) ||
        !perftest::check_range(seen, total * sizeof(unsigned int)) ||
        !perftest::check_range(chain, total * sizeof(unsigned long long)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    hipLaunchKernelGGL(amo_contend_kernel, dim3((unsigned)blocks, 1, (unsigned)nvshmem_n_pes()),
                       dim3((unsigned)threads), 0, (hipStream_t)stream, words, seen, chain, home);
    return perftest::launch_status("amo_contend");
}

}  // extern "C"
