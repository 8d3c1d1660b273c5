// Typed, sized and strided forms of the host-initiated RMA calls, blocking and on a stream, plus
// the typed waits on a stream.  All of them reduce to a copy to/from the translated address, as in
// the reference (src/host/comm/putget.cpp:48-185 for contiguous and strided transfers,
// src/host/comm/sync.cpp:17-58 and src/include/internal/non_abi/nvshmemi_h_to_d_sync_defs.cuh:31-70
// for the waits).  Declarations: reference src/include/host/nvshmem_api.h:199-353 and
// src/include/host/nvshmemx_api.h:94-275.
#include <cstring>
#include <mutex>
#include <type_traits>

#include "nvshmem.h"
#include "runtime.hpp"

namespace nvshmem_amd {
namespace {

bool strided_target(Runtime &rt, const char *what, const void *sym, ptrdiff_t stride, size_t nelems,
                    size_t es, int pe, char **out) {
    if (!rt.initialized) {
        set_error("%s called before nvshmem_init", what);
        return false;
    }
    if (pe < 0 || pe >= rt.npes) {
        set_error("%s: pe %d outside [0, %d)", what, pe, rt.npes);
        return false;
    }
    if (stride < 1) {
        set_error("%s: stride %td must be at least 1", what, stride);
        return false;
    }
    uint64_t off = 0;
    const uint64_t span = nelems ? ((uint64_t)(nelems - 1) * (uint64_t)stride + 1) * es : 0;
    if (!check_symmetric_range(rt, what, sym, span, &off)) return false;
    *out = rt.slice(pe) + off;
    return true;
}

// element i of the source (stride sst) -> element i*dst of the destination
void strided_copy(char *dst, ptrdiff_t dst_stride, const char *src, ptrdiff_t src_stride, size_t nelems,
                  size_t es, hipStream_t stream) {
    if (nelems == 0) return;
    NVSHMEM_AMD_HIP_CHECK(hipMemcpy2DAsync(dst, (size_t)dst_stride * es, src, (size_t)src_stride * es, es,
                                           nelems, hipMemcpyDefault, stream));
}

void iput_on_stream(void *dest, const void *source, ptrdiff_t dst, ptrdiff_t sst, size_t nelems,
                    size_t es, int pe, hipStream_t stream) {
    Runtime &rt = Runtime::get();
    char *target = nullptr;
    if (sst < 1) {
        set_error("iput: source stride %td must be at least 1", sst);
        return;
    }
    if (!strided_target(rt, "iput", dest, dst, nelems, es, pe, &target)) return;
    strided_copy(target, dst, (const char *)source, sst, nelems, es, stream);
}

void iget_on_stream(void *dest, const void *source, ptrdiff_t dst, ptrdiff_t sst, size_t nelems,
                    size_t es, int pe, hipStream_t stream) {
    Runtime &rt = Runtime::get();
    char *target = nullptr;
    if (dst < 1) {
        set_error("iget: destination stride %td must be at least 1", dst);
        return;
    }
    if (!strided_target(rt, "iget", source, sst, nelems, es, pe, &target)) return;
    strided_copy((char *)dest, dst, target, sst, nelems, es, stream);
}

// scalar p: the value travels in the kernel arguments, so the store is stream ordered
__global__ void scalar_p_kernel(void *dest, uint64_t bits, int bytes, int pe) {
    switch (bytes) {
        case 1: nvshmemi_p<uint8_t>((uint8_t *)dest, (uint8_t)bits, pe); break;
        case 2: nvshmemi_p<uint16_t>((uint16_t *)dest, (uint16_t)bits, pe); break;
        case 4: nvshmemi_p<uint32_t>((uint32_t *)dest, (uint32_t)bits, pe); break;
        default: nvshmemi_p<uint64_t>((uint64_t *)dest, bits, pe); break;
    }
}

void p_on_stream(void *dest, const void *value, size_t es, int pe, hipStream_t stream) {
    Runtime &rt = Runtime::get();
    uint64_t off = 0;
    if (!rt.initialized || pe < 0 || pe >= rt.npes) {
        set_error("p: not initialised or pe %d outside [0, %d)", pe, rt.npes);
        return;
    }
    if (!check_symmetric_range(rt, "p", dest, es, &off)) return;
    uint64_t bits = 0;
    memcpy(&bits, value, es);
    hipLaunchKernelGGL(scalar_p_kernel, dim3(1), dim3(1), 0, stream, dest, bits, (int)es, pe);
    NVSHMEM_AMD_HIP_CHECK(hipGetLastError());
}

void g_on_stream(void *value_out, const void *source, size_t es, int pe, hipStream_t stream) {
    memset(value_out, 0, es);
    nvshmemx_getmem_on_stream(value_out, source, es, pe, (nvshmemx_stream_t)stream);
    NVSHMEM_AMD_HIP_CHECK(hipStreamSynchronize(stream));
}

template <typename T>
__global__ void wait_until_kernel(T *ivar, int cmp, T value) {
    nvshmemi_wait_until<T>(ivar, cmp, value);
}
template <typename T>
__global__ void wait_until_all_kernel(T *ivars, size_t nelems, const int *status, int cmp, T value) {
    for (size_t i = threadIdx.x; i < nelems; i += blockDim.x)
        if (!status || !status[i]) nvshmemi_wait_until<T>(ivars + i, cmp, value);
}

template <typename T>
void wait_until_on_stream(T *ivar, int cmp, T value, hipStream_t stream) {
    Runtime &rt = Runtime::get();
    uint64_t off = 0;
    if (!rt.initialized || !check_symmetric_range(rt, "wait_until_on_stream", ivar, sizeof(T), &off)) return;
    if (cmp < NVSHMEM_CMP_EQ || cmp > NVSHMEM_CMP_GE) {
        set_error("wait_until_on_stream: unknown comparison %d", cmp);
        return;
    }
    hipLaunchKernelGGL(wait_until_kernel<T>, dim3(1), dim3(1), 0, stream, ivar, cmp, value);
    NVSHMEM_AMD_HIP_CHECK(hipGetLastError());
}

template <typename T>
void wait_until_all_on_stream(T *ivars, size_t nelems, const int *status, int cmp, T value,
                              hipStream_t stream) {
    Runtime &rt = Runtime::get();
    uint64_t off = 0;
    if (nelems == 0 || !rt.initialized ||
        !check_symmetric_range(rt, "wait_until_all_on_stream", ivars, nelems * sizeof(T), &off))
        return;
    if (cmp < NVSHMEM_CMP_EQ || cmp > NVSHMEM_CMP_GE) {
        set_error("wait_until_all_on_stream: unknown comparison %d", cmp);
        return;
    }
    // `status` is read by the kernel: it must be device-accessible memory (or NULL), as in the reference
    hipLaunchKernelGGL(wait_until_all_kernel<T>, dim3(1), dim3(64), 0, stream, ivars, nelems, status, cmp,
                       value);
    NVSHMEM_AMD_HIP_CHECK(hipGetLastError());
}

template <typename T>
__global__ void wait_until_all_vector_kernel(T *ivars, size_t nelems, const int *status, int cmp,
                                             const T *values) {
    for (size_t i = threadIdx.x; i < nelems; i += blockDim.x)
        if (!status || !status[i]) nvshmemi_wait_until<T>(ivars + i, cmp, values[i]);
}

// `status` and `cmp_values` are read by the kernel: device-accessible memory, as in the reference
// (src/include/internal/non_abi/nvshmemi_h_to_d_sync_defs.cuh:52-70)
template <typename T>
void wait_until_all_vector_on_stream(T *ivars, size_t nelems, const int *status, int cmp, const T *values,
                                     hipStream_t stream) {
    Runtime &rt = Runtime::get();
    uint64_t off = 0;
    if (nelems == 0 || !rt.initialized ||
        !check_symmetric_range(rt, "wait_until_all_vector_on_stream", ivars, nelems * sizeof(T), &off))
        return;
    if (cmp < NVSHMEM_CMP_EQ || cmp > NVSHMEM_CMP_GE) {
        set_error("wait_until_all_vector_on_stream: unknown comparison %d", cmp);
        return;
    }
    if (!values) {
        set_error("wait_until_all_vector_on_stream: cmp_values is NULL");
        return;
    }
    hipLaunchKernelGGL(wait_until_all_vector_kernel<T>, dim3(1), dim3(64), 0, stream, ivars, nelems, status,
                       cmp, values);
    NVSHMEM_AMD_HIP_CHECK(hipGetLastError());
}

void sync0() { NVSHMEM_AMD_HIP_CHECK(hipStreamSynchronize(nullptr)); }

// Host-initiated atomics: one thread applies the device-side operation and leaves what it fetched in
// a pinned word that the host reads after the stream has drained.
template <typename T>
__global__ void host_amo_kernel(int op, T *target, T value, T cond, int pe, T *fetched) {
    T r = T(0);
    switch (op) {
        case NVSHMEMI_AMO_FETCH: r = nvshmemi_atomic_fetch<T>(target, pe); break;
        case NVSHMEMI_AMO_SET: nvshmemi_atomic_set<T>(target, value, pe); break;
        case NVSHMEMI_AMO_SWAP: r = nvshmemi_atomic_swap<T>(target, value, pe); break;
        default:
            if constexpr (!std::is_floating_point<T>::value) {
                switch (op) {
                    case NVSHMEMI_AMO_COMPARE_SWAP: r = nvshmemi_atomic_compare_swap<T>(target, cond, value, pe); break;
                    case NVSHMEMI_AMO_FETCH_ADD: r = nvshmemi_atomic_fetch_add<T>(target, value, pe); break;
                    case NVSHMEMI_AMO_FETCH_AND: r = nvshmemi_atomic_fetch_and<T>(target, value, pe); break;
                    case NVSHMEMI_AMO_FETCH_OR: r = nvshmemi_atomic_fetch_or<T>(target, value, pe); break;
                    case NVSHMEMI_AMO_FETCH_XOR: r = nvshmemi_atomic_fetch_xor<T>(target, value, pe); break;
                    default: break;
                }
            }
            break;
    }
    *fetched = r;
}

template <typename T>
T host_amo(const char *what, int op, const T *target, T value, T cond, int pe) {
    Runtime &rt = Runtime::get();
    std::lock_guard<std::recursive_mutex> lock(rt.mu);
    uint64_t off = 0;
    if (!rt.initialized) {
        set_error("%s called before nvshmem_init", what);
        return T(0);
    }
    if (pe < 0 || pe >= rt.npes) {
        set_error("%s: pe %d outside [0, %d)", what, pe, rt.npes);
        return T(0);
    }
    if (!check_symmetric_range(rt, what, target, sizeof(T), &off)) return T(0);
    if (off % sizeof(T)) {
        set_error("%s: target is not aligned to its type", what);
        return T(0);
    }
    static uint64_t *slot = nullptr;  // pinned, lives until the process ends
    if (!slot) NVSHMEM_AMD_HIP_CHECK(hipHostMalloc((void **)&slot, sizeof(uint64_t), hipHostMallocDefault));
    *slot = 0;
    hipLaunchKernelGGL(host_amo_kernel<T>, dim3(1), dim3(1), 0, nullptr, op, const_cast<T *>(target), value, cond,
                       pe, reinterpret_cast<T *>(slot));
    NVSHMEM_AMD_HIP_CHECK(hipGetLastError());
    sync0();
    T out;
    memcpy(&out, slot, sizeof(T));
    return out;
}

}  // namespace
}  // namespace nvshmem_amd

using namespace nvshmem_amd;

extern "C" {

uint64_t nvshmem_signal_fetch(uint64_t *sig_addr) {
    uint64_t v = 0;
    nvshmemx_getmem_on_stream(&v, sig_addr, sizeof v, 0, nullptr);
    sync0();
    return v;
}

#define NVSHMEMI_DEFINE_TYPED_HOST_RMA(NAME, TYPE, TAG)                                           \
    void nvshmemx_##NAME##_p_on_stream(TYPE *dest, const TYPE value, int pe, nvshmemx_stream_t s) { \
        p_on_stream(dest, &value, sizeof(TYPE), pe, (hipStream_t)s);                              \
    }                                                                                             \
    void nvshmem_##NAME##_p(TYPE *dest, const TYPE value, int pe) {                               \
        p_on_stream(dest, &value, sizeof(TYPE), pe, nullptr);                                     \
        sync0();                                                                                  \
    }                                                                                             \
    TYPE nvshmemx_##NAME##_g_on_stream(const TYPE *src, int pe, nvshmemx_stream_t s) {            \
        TYPE v;                                                                                   \
        g_on_stream(&v, src, sizeof(TYPE), pe, (hipStream_t)s);                                   \
        return v;                                                                                 \
    }                                                                                             \
    TYPE nvshmem_##NAME##_g(const TYPE *src, int pe) {                                            \
        TYPE v;                                                                                   \
        g_on_stream(&v, src, sizeof(TYPE), pe, nullptr);                                          \
        return v;                                                                                 \
    }                                                                                             \
    void nvshmemx_##NAME##_put_nbi_on_stream(TYPE *dest, const TYPE *source, size_t nelems,       \
                                             int pe, nvshmemx_stream_t s) {                       \
        nvshmemx_putmem_on_stream(dest, source, nelems * sizeof(TYPE), pe, s);                    \
    }                                                                                             \
    void nvshmemx_##NAME##_get_nbi_on_stream(TYPE *dest, const TYPE *source, size_t nelems,       \
                                             int pe, nvshmemx_stream_t s) {                       \
        nvshmemx_getmem_on_stream(dest, source, nelems * sizeof(TYPE), pe, s);                    \
    }                                                                                             \
    void nvshmem_##NAME##_put_nbi(TYPE *dest, const TYPE *source, size_t nelems, int pe) {        \
        nvshmemx_putmem_on_stream(dest, source, nelems * sizeof(TYPE), pe, nullptr);              \
    }                                                                                             \
    void nvshmem_##NAME##_get_nbi(TYPE *dest, const TYPE *source, size_t nelems, int pe) {        \
        nvshmemx_getmem_on_stream(dest, source, nelems * sizeof(TYPE), pe, nullptr);              \
    }                                                                                             \
    void nvshmemx_##NAME##_iput_on_stream(TYPE *dest, const TYPE *source, ptrdiff_t dst,          \
                                          ptrdiff_t sst, size_t nelems, int pe,                   \
                                          nvshmemx_stream_t s) {                                  \
        iput_on_stream(dest, source, dst, sst, nelems, sizeof(TYPE), pe, (hipStream_t)s);         \
    }                                                                                             \
    void nvshmemx_##NAME##_iget_on_stream(TYPE *dest, const TYPE *source, ptrdiff_t dst,          \
                                          ptrdiff_t sst, size_t nelems, int pe,                   \
                                          nvshmemx_stream_t s) {                                  \
        iget_on_stream(dest, source, dst, sst, nelems, sizeof(TYPE), pe, (hipStream_t)s);         \
    }                                                                                             \
    void nvshmem_##NAME##_iput(TYPE *dest, const TYPE *source, ptrdiff_t dst, ptrdiff_t sst,      \
                               size_t nelems, int pe) {                                           \
        iput_on_stream(dest, source, dst, sst, nelems, sizeof(TYPE), pe, nullptr);                \
        sync0();                                                                                  \
    }                                                                                             \
    void nvshmem_##NAME##_iget(TYPE *dest, const TYPE *source, ptrdiff_t dst, ptrdiff_t sst,      \
                               size_t nelems, int pe) {                                           \
        iget_on_stream(dest, source, dst, sst, nelems, sizeof(TYPE), pe, nullptr);                \
        sync0();                                                                                  \
    }                                                                                             \
    void nvshmemx_##NAME##_put_signal_on_stream(TYPE *dest, const TYPE *source, size_t nelems,    \
                                                uint64_t *sig_addr, uint64_t signal, int sig_op,  \
                                                int pe, nvshmemx_stream_t s) {                    \
        nvshmemx_putmem_signal_on_stream(dest, source, nelems * sizeof(TYPE), sig_addr, signal,   \
                                         sig_op, pe, s);                                          \
    }                                                                                             \
    void nvshmemx_##NAME##_put_signal_nbi_on_stream(TYPE *dest, const TYPE *source,               \
                                                    size_t nelems, uint64_t *sig_addr,            \
                                                    uint64_t signal, int sig_op, int pe,          \
                                                    nvshmemx_stream_t s) {                        \
        nvshmemx_putmem_signal_on_stream(dest, source, nelems * sizeof(TYPE), sig_addr, signal,   \
                                         sig_op, pe, s);                                          \
    }
NVSHMEMI_REPT_FOR_STANDARD_RMA_TYPES(NVSHMEMI_DEFINE_TYPED_HOST_RMA)
#undef NVSHMEMI_DEFINE_TYPED_HOST_RMA

#define NVSHMEMI_DEFINE_SIZED_HOST_RMA(BITS, BYTES)                                               \
    void nvshmemx_put##BITS##_on_stream(void *dest, const void *source, size_t nelems, int pe,    \
                                        nvshmemx_stream_t s) {                                    \
        nvshmemx_putmem_on_stream(dest, source, nelems * BYTES, pe, s);                           \
    }                                                                                             \
    void nvshmemx_get##BITS##_on_stream(void *dest, const void *source, size_t nelems, int pe,    \
                                        nvshmemx_stream_t s) {                                    \
        nvshmemx_getmem_on_stream(dest, source, nelems * BYTES, pe, s);                           \
    }                                                                                             \
    void nvshmemx_put##BITS##_nbi_on_stream(void *dest, const void *source, size_t nelems,        \
                                            int pe, nvshmemx_stream_t s) {                        \
        nvshmemx_putmem_on_stream(dest, source, nelems * BYTES, pe, s);                           \
    }                                                                                             \
    void nvshmemx_get##BITS##_nbi_on_stream(void *dest, const void *source, size_t nelems,        \
                                            int pe, nvshmemx_stream_t s) {                        \
        nvshmemx_getmem_on_stream(dest, source, nelems * BYTES, pe, s);                           \
    }                                                                                             \
    void nvshmem_put##BITS(void *dest, const void *source, size_t nelems, int pe) {               \
        nvshmem_putmem(dest, source, nelems * BYTES, pe);                                         \
    }                                                                                             \
    void nvshmem_get##BITS(void *dest, const void *source, size_t nelems, int pe) {               \
        nvshmem_getmem(dest, source, nelems * BYTES, pe);                                         \
    }                                                                                             \
    void nvshmem_put##BITS##_nbi(void *dest, const void *source, size_t nelems, int pe) {         \
        nvshmemx_putmem_on_stream(dest, source, nelems * BYTES, pe, nullptr);                     \
    }                                                                                             \
    void nvshmem_get##BITS##_nbi(void *dest, const void *source, size_t nelems, int pe) {         \
        nvshmemx_getmem_on_stream(dest, source, nelems * BYTES, pe, nullptr);                     \
    }                                                                                             \
    void nvshmemx_iput##BITS##_on_stream(void *dest, const void *source, ptrdiff_t dst,           \
                                         ptrdiff_t sst, size_t nelems, int pe,                    \
                                         nvshmemx_stream_t s) {                                   \
        iput_on_stream(dest, source, dst, sst, nelems, BYTES, pe, (hipStream_t)s);                \
    }                                                                                             \
    void nvshmemx_iget##BITS##_on_stream(void *dest, const void *source, ptrdiff_t dst,           \
                                         ptrdiff_t sst, size_t nelems, int pe,                    \
                                         nvshmemx_stream_t s) {                                   \
        iget_on_stream(dest, source, dst, sst, nelems, BYTES, pe, (hipStream_t)s);                \
    }                                                                                             \
    void nvshmem_iput##BITS(void *dest, const void *source, ptrdiff_t dst, ptrdiff_t sst,         \
                            size_t nelems, int pe) {                                              \
        iput_on_stream(dest, source, dst, sst, nelems, BYTES, pe, nullptr);                       \
        sync0();                                                                                  \
    }                                                                                             \
    void nvshmem_iget##BITS(void *dest, const void *source, ptrdiff_t dst, ptrdiff_t sst,         \
                            size_t nelems, int pe) {                                              \
        iget_on_stream(dest, source, dst, sst, nelems, BYTES, pe, nullptr);                       \
        sync0();                                                                                  \
    }                                                                                             \
    void nvshmemx_put##BITS##_signal_on_stream(void *dest, const void *source, size_t nelems,     \
                                               uint64_t *sig_addr, uint64_t signal, int sig_op,   \
                                               int pe, nvshmemx_stream_t s) {                     \
        nvshmemx_putmem_signal_on_stream(dest, source, nelems * BYTES, sig_addr, signal, sig_op,  \
                                         pe, s);                                                  \
    }                                                                                             \
    void nvshmemx_put##BITS##_signal_nbi_on_stream(void *dest, const void *source,                \
                                                   size_t nelems, uint64_t *sig_addr,             \
                                                   uint64_t signal, int sig_op, int pe,           \
                                                   nvshmemx_stream_t s) {                         \
        nvshmemx_putmem_signal_on_stream(dest, source, nelems * BYTES, sig_addr, signal, sig_op,  \
                                         pe, s);                                                  \
    }
NVSHMEMI_REPT_FOR_SIZES(NVSHMEMI_DEFINE_SIZED_HOST_RMA)
#undef NVSHMEMI_DEFINE_SIZED_HOST_RMA

#define NVSHMEMI_DEFINE_WAIT_ON_STREAM(NAME, TYPE)                                                \
    void nvshmemx_##NAME##_wait_until_on_stream(TYPE *ivar, int cmp, TYPE cmp_value,              \
                                                nvshmemx_stream_t s) {                            \
        wait_until_on_stream<TYPE>(ivar, cmp, cmp_value, (hipStream_t)s);                         \
    }                                                                                             \
    void nvshmemx_##NAME##_wait_until_all_on_stream(TYPE *ivars, size_t nelems,                   \
                                                    const int *status, int cmp, TYPE cmp_value,   \
                                                    nvshmemx_stream_t s) {                        \
        wait_until_all_on_stream<TYPE>(ivars, nelems, status, cmp, cmp_value, (hipStream_t)s);    \
    }
NVSHMEMI_REPT_FOR_WAIT_TYPES(NVSHMEMI_DEFINE_WAIT_ON_STREAM)
#undef NVSHMEMI_DEFINE_WAIT_ON_STREAM

#define NVSHMEMI_DEFINE_WAIT_VECTOR_ON_STREAM(NAME, TYPE)                                         \
    void nvshmemx_##NAME##_wait_until_all_vector_on_stream(TYPE *ivars, size_t nelems,            \
                                                           const int *status, int cmp,            \
                                                           TYPE *cmp_values, nvshmemx_stream_t s) { \
        wait_until_all_vector_on_stream<TYPE>(ivars, nelems, status, cmp, cmp_values, (hipStream_t)s); \
    }
NVSHMEMI_REPT_FOR_WAIT_TYPES(NVSHMEMI_DEFINE_WAIT_VECTOR_ON_STREAM)
#undef NVSHMEMI_DEFINE_WAIT_VECTOR_ON_STREAM

#define NVSHMEMI_DEFINE_AMO_FETCH_SET_SWAP_HOST(NAME, TYPE)                                       \
    TYPE nvshmem_##NAME##_atomic_fetch(const TYPE *target, int pe) {                              \
        return host_amo<TYPE>("nvshmem_" #NAME "_atomic_fetch", NVSHMEMI_AMO_FETCH, target, (TYPE)0, (TYPE)0, pe); \
    }                                                                                             \
    void nvshmem_##NAME##_atomic_set(TYPE *target, TYPE value, int pe) {                          \
        (void)host_amo<TYPE>("nvshmem_" #NAME "_atomic_set", NVSHMEMI_AMO_SET, target, value, (TYPE)0, pe); \
    }                                                                                             \
    TYPE nvshmem_##NAME##_atomic_swap(TYPE *target, TYPE value, int pe) {                         \
        return host_amo<TYPE>("nvshmem_" #NAME "_atomic_swap", NVSHMEMI_AMO_SWAP, target, value, (TYPE)0, pe); \
    }
NVSHMEMI_REPT_FOR_STANDARD_AMO_TYPES(NVSHMEMI_DEFINE_AMO_FETCH_SET_SWAP_HOST)
NVSHMEMI_REPT_FOR_EXTENDED_AMO_TYPES(NVSHMEMI_DEFINE_AMO_FETCH_SET_SWAP_HOST)
#undef NVSHMEMI_DEFINE_AMO_FETCH_SET_SWAP_HOST

#define NVSHMEMI_DEFINE_AMO_ARITH_HOST(NAME, TYPE)                                                \
    TYPE nvshmem_##NAME##_atomic_compare_swap(TYPE *target, TYPE cond, TYPE value, int pe) {      \
        return host_amo<TYPE>("nvshmem_" #NAME "_atomic_compare_swap", NVSHMEMI_AMO_COMPARE_SWAP, target, value, cond, pe); \
    }                                                                                             \
    TYPE nvshmem_##NAME##_atomic_fetch_add(TYPE *target, TYPE value, int pe) {                    \
        return host_amo<TYPE>("nvshmem_" #NAME "_atomic_fetch_add", NVSHMEMI_AMO_FETCH_ADD, target, value, (TYPE)0, pe); \
    }                                                                                             \
    void nvshmem_##NAME##_atomic_add(TYPE *target, TYPE value, int pe) {                          \
        (void)host_amo<TYPE>("nvshmem_" #NAME "_atomic_add", NVSHMEMI_AMO_FETCH_ADD, target, value, (TYPE)0, pe); \
    }                                                                                             \
    TYPE nvshmem_##NAME##_atomic_fetch_inc(TYPE *target, int pe) {                                \
        return host_amo<TYPE>("nvshmem_" #NAME "_atomic_fetch_inc", NVSHMEMI_AMO_FETCH_ADD, target, (TYPE)1, (TYPE)0, pe); \
    }                                                                                             \
    void nvshmem_##NAME##_atomic_inc(TYPE *target, int pe) {                                      \
        (void)host_amo<TYPE>("nvshmem_" #NAME "_atomic_inc", NVSHMEMI_AMO_FETCH_ADD, target, (TYPE)1, (TYPE)0, pe); \
    }
NVSHMEMI_REPT_FOR_STANDARD_AMO_TYPES(NVSHMEMI_DEFINE_AMO_ARITH_HOST)
#undef NVSHMEMI_DEFINE_AMO_ARITH_HOST

#define NVSHMEMI_DEFINE_AMO_BITWISE_HOST(NAME, TYPE)                                              \
    TYPE nvshmem_##NAME##_atomic_fetch_and(TYPE *target, TYPE value, int pe) {                    \
        return host_amo<TYPE>("nvshmem_" #NAME "_atomic_fetch_and", NVSHMEMI_AMO_FETCH_AND, target, value, (TYPE)0, pe); \
    }                                                                                             \
    TYPE nvshmem_##NAME##_atomic_fetch_or(TYPE *target, TYPE value, int pe) {                     \
        return host_amo<TYPE>("nvshmem_" #NAME "_atomic_fetch_or", NVSHMEMI_AMO_FETCH_OR, target, value, (TYPE)0, pe); \
    }                                                                                             \
    TYPE nvshmem_##NAME##_atomic_fetch_xor(TYPE *target, TYPE value, int pe) {                    \
        return host_amo<TYPE>("nvshmem_" #NAME "_atomic_fetch_xor", NVSHMEMI_AMO_FETCH_XOR, target, value, (TYPE)0, pe); \
    }                                                                                             \
    void nvshmem_##NAME##_atomic_and(TYPE *target, TYPE value, int pe) {                          \
        (void)host_amo<TYPE>("nvshmem_" #NAME "_atomic_and", NVSHMEMI_AMO_FETCH_AND, target, value, (TYPE)0, pe); \
    }                                                                                             \
    void nvshmem_##NAME##_atomic_or(TYPE *target, TYPE value, int pe) {                           \
        (void)host_amo<TYPE>("nvshmem_" #NAME "_atomic_or", NVSHMEMI_AMO_FETCH_OR, target, value, (TYPE)0, pe); \
    }                                                                                             \
    void nvshmem_##NAME##_atomic_xor(TYPE *target, TYPE value, int pe) {                          \
        (void)host_amo<TYPE>("nvshmem_" #NAME "_atomic_xor", NVSHMEMI_AMO_FETCH_XOR, target, value, (TYPE)0, pe); \
    }
NVSHMEMI_REPT_FOR_BITWISE_AMO_TYPES(NVSHMEMI_DEFINE_AMO_BITWISE_HOST)
#undef NVSHMEMI_DEFINE_AMO_BITWISE_HOST

}  // extern "C"
