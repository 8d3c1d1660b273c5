/*
 * CPU oracle of the NVSHMEM data-movement path.  TEST INFRASTRUCTURE ONLY (see nvshmem_oracle.h).
 * Plain C loops; the large ones are split over OpenMP threads so full-size configurations finish
 * in seconds.  Compiled with -ffp-contract=off so no multiply-add is fused.
 */
#include "nvshmem_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static const size_t k_dtype_size[ORC_DT_COUNT] = {1, 2, 4, 8, 1, 2, 4, 8, 2, 2, 4, 8};
size_t oracle_dtype_size(int dtype) {
    return (dtype >= 0 && dtype < ORC_DT_COUNT) ? k_dtype_size[dtype] : 0;
}

void oracle_set_threads(int nthreads) {
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#else
    (void)nthreads;
#endif
}
int oracle_get_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------------- */
/* seeded inputs                                                                                */
/* ------------------------------------------------------------------------------------------- */
uint64_t oracle_splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

uint64_t oracle_rand_u64(uint64_t seed, uint64_t pe, uint64_t index) {
    const uint64_t stream = oracle_splitmix64(seed ^ (pe * 0xD1B54A32D192ED03ull + 0x2545F4914F6CDD1Dull));
    return oracle_splitmix64(stream + index * 0x9E3779B97F4A7C15ull);
}

void oracle_fill_u64(uint64_t *out, size_t n, uint64_t seed, uint64_t pe) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) out[i] = oracle_rand_u64(seed, pe, i);
}

void oracle_fill_bytes(uint8_t *out, size_t n, uint64_t seed, uint64_t pe) {
    const size_t words = n / 8;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < words; ++i) {
        const uint64_t r = oracle_rand_u64(seed, pe, i);
        memcpy(out + 8 * i, &r, 8);
    }
    if (n % 8) {
        const uint64_t r = oracle_rand_u64(seed, pe, words);
        memcpy(out + 8 * words, &r, n % 8);
    }
}

void oracle_fill_i32_pm2p20(int32_t *out, size_t n, uint64_t seed, uint64_t pe) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i)
        out[i] = (int32_t)(oracle_rand_u64(seed, pe, i) % ((1u << 21) + 1u)) - (1 << 20);
}

/* one standard normal per index: Box-Muller on two uniforms derived from (seed, pe, index) */
static double normal_at(uint64_t seed, uint64_t pe, uint64_t i) {
    const uint64_t a = oracle_rand_u64(seed, pe, 2 * i);
    const uint64_t b = oracle_rand_u64(seed, pe, 2 * i + 1);
    const double u1 = ((double)(a >> 11) + 1.0) * (1.0 / 9007199254740993.0); /* (0, 1) */
    const double u2 = (double)(b >> 11) * (1.0 / 9007199254740992.0);         /* [0, 1) */
    return sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
}

void oracle_fill_f32_normal(float *out, size_t n, uint64_t seed, uint64_t pe) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) out[i] = (float)normal_at(seed, pe, i);
}
void oracle_fill_bf16_normal(uint16_t *out, size_t n, uint64_t seed, uint64_t pe) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) out[i] = oracle_f32_to_bf16((float)normal_at(seed, pe, i));
}
void oracle_fill_f16_normal(uint16_t *out, size_t n, uint64_t seed, uint64_t pe) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) out[i] = oracle_f32_to_f16((float)normal_at(seed, pe, i));
}

/* ------------------------------------------------------------------------------------------- */
/* 16-bit floats                                                                                */
/* ------------------------------------------------------------------------------------------- */
static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float oracle_bf16_to_f32(uint16_t v) { return bits_f32((uint32_t)v << 16); }

uint16_t oracle_f32_to_bf16(float f) {
    const uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

float oracle_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0x1f) return bits_f32(sign | 0x7f800000u | (man << 13));
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        int e = -1; /* normalise the subnormal */
        do { man <<= 1; ++e; } while (!(man & 0x400u));
        return bits_f32(sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13));
    }
    return bits_f32(sign | ((exp + 127 - 15) << 23) | (man << 13));
}

uint16_t oracle_f32_to_f16(float f) {
    const uint32_t u = f32_bits(f);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t abs = u & 0x7fffffffu;
    if (abs > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((abs >> 13) & 0x3ffu));
    if (abs >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* rounds to infinity */
    if (abs < 0x33000001u) return sign;                        /* rounds to zero (<= 2^-25) */
    int exp = (int)(abs >> 23) - 127;
    uint32_t man = (abs & 0x7fffffu) | 0x800000u;
    int shift;
    uint32_t half_exp;
    if (exp < -14) { shift = 13 + (-14 - exp); half_exp = 0; }
    else { shift = 13; half_exp = (uint32_t)(exp + 15); }
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
    /* q carries the implicit bit for normals: adding it to the exponent field also handles the
     * mantissa overflow into the next exponent */
    if (half_exp == 0) return (uint16_t)(sign | q);
    return (uint16_t)(sign | (((half_exp - 1) << 10) + q));
}

/* ------------------------------------------------------------------------------------------- */
/* point to point                                                                               */
/* put: reference nvshmemi_put, src/include/non_abi/device/common/nvshmemi_common_device.cuh:488-505
 * get: :429-446; both are a byte copy between the caller's buffer and the target PE's copy.    */
/* ------------------------------------------------------------------------------------------- */
void oracle_copy(void *dst, const void *src, size_t bytes) { memmove(dst, src, bytes); }

/* ring pattern of the reference's put example (examples/put-block.cu:39, :93-104); the copies are
 * cut into 1 MiB pieces so that the threads set with oracle_set_threads share them */
#define ORC_RING_PIECE ((size_t)1 << 20)
static void ring_copy(uint8_t *dst, const uint8_t *src, int npes, size_t bytes, int dst_step, int src_step) {
    const long pieces = (long)((bytes + ORC_RING_PIECE - 1) / ORC_RING_PIECE);
#pragma omp parallel for collapse(2) schedule(static)
    for (int p = 0; p < npes; ++p)
        for (long k = 0; k < pieces; ++k) {
            const size_t off = (size_t)k * ORC_RING_PIECE;
            const size_t len = bytes - off < ORC_RING_PIECE ? bytes - off : ORC_RING_PIECE;
            memcpy(dst + (size_t)((p + dst_step) % npes) * bytes + off, src + (size_t)((p + src_step) % npes) * bytes + off,
                   len);
        }
}
void oracle_ring_put(uint8_t *dst, const uint8_t *src, int npes, size_t bytes) {
    ring_copy(dst, src, npes, bytes, 1, 0);
}
void oracle_ring_get(uint8_t *dst, const uint8_t *src, int npes, size_t bytes) {
    ring_copy(dst, src, npes, bytes, 0, 1);
}

/* reference nvshmemi_signal_op, nvshmemi_common_device.cuh:507-527; SET = 9, ADD = 10
 * (src/include/device_host_transport/nvshmem_common_transport.h:39) */
uint64_t oracle_signal_op(uint64_t current, uint64_t signal, int sig_op) {
    if (sig_op == 9) return signal;
    if (sig_op == 10) return current + signal;
    return current;
}

/* reference comparators, src/include/non_abi/device/wait/nvshmemi_wait_until_apis.cuh:37-155 with
 * the enum order EQ NE GT LE LT GE of nvshmem_constants.h:48-56 */
int oracle_compare_u64(uint64_t found, int cmp, uint64_t expected) {
    switch (cmp) {
        case 0: return found == expected;
        case 1: return found != expected;
        case 2: return found > expected;
        case 3: return found <= expected;
        case 4: return found < expected;
        case 5: return found >= expected;
        default: return 1;
    }
}
int oracle_compare_i64(int64_t found, int cmp, int64_t expected) {
    switch (cmp) {
        case 0: return found == expected;
        case 1: return found != expected;
        case 2: return found > expected;
        case 3: return found <= expected;
        case 4: return found < expected;
        case 5: return found >= expected;
        default: return 1;
    }
}

/* reference nvshmemi_ptr, nvshmemi_common_device.cuh:578-590 / src/host/mem/mem_heap.cpp:2373-2385:
 * NULL unless 0 <= pe < npes and ptr inside the heap; else peer base + offset.  With logical PEs the
 * "heap" a pointer may lie in is any PE's slice, and the offset is taken inside that slice. */
uint64_t oracle_ptr(uint64_t heap_base, uint64_t heap_size, int npes, uint64_t ptr, int pe) {
    if (pe < 0 || pe >= npes || ptr < heap_base) return 0;
    const uint64_t d = ptr - heap_base;
    if (d >= heap_size * (uint64_t)npes) return 0;
    return heap_base + (uint64_t)pe * heap_size + d % heap_size;
}

/* ------------------------------------------------------------------------------------------- */
/* reduce                                                                                       */
/* element operator: reference perform_gpu_rdxn, src/include/non_abi/device/coll/reduce.cuh:49-105
 * fold order: reference gather-then-fold path, reduce.cuh:1297-1303:
 *     acc = op(x[0], x[1]);  acc = op(x[i], acc)  for i = 2 .. npes-1                            */
/* ------------------------------------------------------------------------------------------- */
#define DEFINE_INT_OPS(NAME, T, U)                                                   \
    static T NAME##_apply(int op, T a, T b) {                                        \
        switch (op) {                                                                \
            case ORC_and: return (T)(a & b);                                         \
            case ORC_or: return (T)(a | b);                                          \
            case ORC_xor: return (T)(a ^ b);                                         \
            case ORC_min: return (a < b) ? a : b;                                    \
            case ORC_max: return (a > b) ? a : b;                                    \
            case ORC_sum: return (T)(U)((U)a + (U)b);                                \
            default: return (T)(U)((U)a * (U)b);                                     \
        }                                                                            \
    }
DEFINE_INT_OPS(i8, int8_t, uint8_t)
DEFINE_INT_OPS(i16, int16_t, uint16_t)
DEFINE_INT_OPS(i32, int32_t, uint32_t)
DEFINE_INT_OPS(i64, int64_t, uint64_t)
DEFINE_INT_OPS(u8, uint8_t, uint8_t)
DEFINE_INT_OPS(u16, uint16_t, uint16_t)
DEFINE_INT_OPS(u32, uint32_t, uint32_t)
DEFINE_INT_OPS(u64, uint64_t, uint64_t)

#define DEFINE_FP_OPS(NAME, T)                                                       \
    static T NAME##_apply(int op, T a, T b) {                                        \
        switch (op) {                                                                \
            case ORC_min: return (a < b) ? a : b;                                    \
            case ORC_max: return (a > b) ? a : b;                                    \
            case ORC_sum: return a + b;                                              \
            default: return a * b;                                                   \
        }                                                                            \
    }
DEFINE_FP_OPS(f32, float)
DEFINE_FP_OPS(f64, double)

/* 16-bit floats: the operation in the element type = exact fp32 operation, one rounding to 16 bits
 * (reference uses the native __nv_bfloat16 / half operators, reduce.cuh:91-99) */
static uint16_t bf16_apply(int op, uint16_t a, uint16_t b) {
    const float fa = oracle_bf16_to_f32(a), fb = oracle_bf16_to_f32(b);
    switch (op) {
        case ORC_min: return (fa < fb) ? a : b;
        case ORC_max: return (fa > fb) ? a : b;
        case ORC_sum: return oracle_f32_to_bf16(fa + fb);
        default: return oracle_f32_to_bf16(fa * fb);
    }
}
static uint16_t f16_apply(int op, uint16_t a, uint16_t b) {
    const float fa = oracle_f16_to_f32(a), fb = oracle_f16_to_f32(b);
    switch (op) {
        case ORC_min: return (fa < fb) ? a : b;
        case ORC_max: return (fa > fb) ? a : b;
        case ORC_sum: return oracle_f32_to_f16(fa + fb);
        default: return oracle_f32_to_f16(fa * fb);
    }
}

#define FOLD_LOOP(NAME, T)                                                           \
    {                                                                                \
        const T *s = (const T *)src;                                                 \
        T *d = (T *)dst;                                                             \
        _Pragma("omp parallel for schedule(static)")                                 \
        for (size_t k = 0; k < nelems; ++k) {                                        \
            T acc = s[k];                                                            \
            if (npes > 1) acc = NAME##_apply(op, acc, s[nelems + k]);                \
            for (int p = 2; p < npes; ++p)                                           \
                acc = NAME##_apply(op, s[(size_t)p * nelems + k], acc);              \
            d[k] = acc;                                                              \
        }                                                                            \
    }                                                                                \
    break;

int oracle_reduce(int dtype, int op, int npes, size_t nelems, const void *src, void *dst) {
    if (op < ORC_and || op > ORC_prod) return -1;
    if (dtype >= ORC_f16 && op < ORC_min) return -1; /* no bitwise ops on floating types */
    switch (dtype) {
        case ORC_i8: FOLD_LOOP(i8, int8_t)
        case ORC_i16: FOLD_LOOP(i16, int16_t)
        case ORC_i32: FOLD_LOOP(i32, int32_t)
        case ORC_i64: FOLD_LOOP(i64, int64_t)
        case ORC_u8: FOLD_LOOP(u8, uint8_t)
        case ORC_u16: FOLD_LOOP(u16, uint16_t)
        case ORC_u32: FOLD_LOOP(u32, uint32_t)
        case ORC_u64: FOLD_LOOP(u64, uint64_t)
        case ORC_f16: FOLD_LOOP(f16, uint16_t)
        case ORC_bf16: FOLD_LOOP(bf16, uint16_t)
        case ORC_f32: FOLD_LOOP(f32, float)
        case ORC_f64: FOLD_LOOP(f64, double)
        default: return -1;
    }
    return 0;
}

/* reducescatter: reference nvshmemi_reducescatter_allpush_threadgroup,
 * src/include/non_abi/device/coll/reducescatter.cuh:36-90: PE q gathers block q of every PE's source
 * and folds it as  acc = op(x0, x1);  acc = op(acc, x_p)  for p = 2 .. npes-1  (:63-86, where
 * gpu_linear_reduce(op1 = dest, op2 = x_p) computes op(dest, x_p)). */
#define SCATTER_LOOP(NAME, T)                                                        \
    {                                                                                \
        const T *s = (const T *)src;                                                 \
        T *d = (T *)dst;                                                             \
        const size_t row = (size_t)npes * nelems;                                    \
        _Pragma("omp parallel for schedule(static)")                                 \
        for (size_t g = 0; g < row; ++g) { /* g = q*nelems + k */                    \
            T acc = s[g];                                                            \
            for (int p = 1; p < npes; ++p) acc = NAME##_apply(op, acc, s[(size_t)p * row + g]); \
            d[g] = acc;                                                              \
        }                                                                            \
    }                                                                                \
    break;

int oracle_reducescatter(int dtype, int op, int npes, size_t nelems, const void *src, void *dst) {
    if (op < ORC_and || op > ORC_prod) return -1;
    if (dtype >= ORC_f16 && op < ORC_min) return -1;
    switch (dtype) {
        case ORC_i8: SCATTER_LOOP(i8, int8_t)
        case ORC_i16: SCATTER_LOOP(i16, int16_t)
        case ORC_i32: SCATTER_LOOP(i32, int32_t)
        case ORC_i64: SCATTER_LOOP(i64, int64_t)
        case ORC_u8: SCATTER_LOOP(u8, uint8_t)
        case ORC_u16: SCATTER_LOOP(u16, uint16_t)
        case ORC_u32: SCATTER_LOOP(u32, uint32_t)
        case ORC_u64: SCATTER_LOOP(u64, uint64_t)
        case ORC_f16: SCATTER_LOOP(f16, uint16_t)
        case ORC_bf16: SCATTER_LOOP(bf16, uint16_t)
        case ORC_f32: SCATTER_LOOP(f32, float)
        case ORC_f64: SCATTER_LOOP(f64, double)
        default: return -1;
    }
    return 0;
}

/* maxloc over (value, location) pairs: operator reference src/include/non_abi/device/coll/reduce.cuh:107-111
 * `(op1.x > op2.x) ? op1 : op2`, folded as in the rooted flat reduce (:1738-1747): acc = source of
 * member 0, then acc = op(acc, source of member i) for i = 1..n-1; all members receive the result.
 * src is [npes][nelems][2] doubles, dst likewise. */
void oracle_maxloc_reduce(int npes, size_t nelems, const double *src, double *dst) {
    for (size_t k = 0; k < nelems; ++k) {
        double v = src[2 * k], loc = src[2 * k + 1];
        for (int p = 1; p < npes; ++p) {
            const double *x = src + ((size_t)p * nelems + k) * 2;
            if (!(v > x[0])) {
                v = x[0];
                loc = x[1];
            }
        }
        for (int q = 0; q < npes; ++q) {
            dst[((size_t)q * nelems + k) * 2] = v;
            dst[((size_t)q * nelems + k) * 2 + 1] = loc;
        }
    }
}

/* broadcast: reference src/include/non_abi/device/coll/broadcast.cuh:276-337 (every PE's dest gets
 * the root's source; the root copies too when dest != source, :97) */
void oracle_broadcast(int npes, size_t bytes, int root, const uint8_t *src, uint8_t *dst) {
    for (int q = 0; q < npes; ++q) memcpy(dst + (size_t)q * bytes, src + (size_t)root * bytes, bytes);
}

/* ------------------------------------------------------------------------------------------- */
/* atomic memory operations: OpenSHMEM semantics of the calls stamped in the reference's
 * src/include/device/nvshmem_defines.h:742-1236 (fetch_add :742-757, fetch_inc :821-836,
 * compare_swap :907-922, fetch_and/or/xor :955-1115, swap :1135-1150, fetch :1184-1196,
 * set :1213-1221); op ids of nvshmemi_amo_t, nvshmem_common_transport.h:41-62.                 */
/* ------------------------------------------------------------------------------------------- */
uint64_t oracle_amo(int op, int bits, uint64_t current, uint64_t value, uint64_t cond,
                    uint64_t *fetched) {
    const uint64_t mask = bits >= 64 ? ~0ull : ((1ull << bits) - 1ull);
    current &= mask;
    value &= mask;
    cond &= mask;
    if (fetched) *fetched = current;
    uint64_t next = current;
    switch (op) {
        case 2: case 13: next = current + 1; break;            /* inc, fetch_inc */
        case 3: case 18: next = value; break;                  /* set, swap */
        case 4: case 14: next = current + value; break;        /* add, fetch_add */
        case 5: case 15: next = current & value; break;        /* and, fetch_and */
        case 6: case 16: next = current | value; break;        /* or, fetch_or */
        case 7: case 17: next = current ^ value; break;        /* xor, fetch_xor */
        case 12: break;                                        /* fetch */
        case 19: next = current == cond ? value : current; break; /* compare_swap */
        default: break;
    }
    return next & mask;
}

/* ------------------------------------------------------------------------------------------- */
/* teams: reference nvshmemi_team_split_strided, src/host/team/team_internal.cpp:2182-2290
 * (argument checks :2197-2222, global triple :2214-2216), nvshmemi_team_split_2d :2292-2349,
 * nvshmemi_team_translate_pe :579-589 (member index wraps modulo the size; an index above the size
 * gives -1).                                                                                   */
/* ------------------------------------------------------------------------------------------- */
int oracle_team_split_strided(const int parent[3], int npes_world, int start, int stride, int size,
                              int child[3]) {
    child[0] = child[1] = child[2] = -1;
    if (start < 0 || start >= parent[2] || size <= 0 || size > parent[2] || stride < 1) return -1;
    const int g_start = parent[0] + start * parent[1];
    const int g_stride = parent[1] * stride;
    const int g_end = g_start + g_stride * (size - 1);
    if (g_start >= npes_world || g_end >= npes_world) return -1;
    child[0] = g_start;
    child[1] = g_stride;
    child[2] = size;
    return 0;
}

int oracle_team_translate_pe(const int src[3], int src_pe, const int dst[3]) {
    if (src_pe < 0 || src_pe > src[2]) return -1;
    const int world = src[0] + (src_pe % src[2]) * src[1];
    const int d = world - dst[0];
    if (d < 0 || d % dst[1] != 0 || d / dst[1] >= dst[2]) return -1;
    return d / dst[1];
}

void oracle_team_split_2d(const int parent[3], int xrange, int index, int xteam[3], int yteam[3]) {
    const int n = parent[2];
    if (xrange > n) xrange = n;
    const int row = index / xrange, col = index % xrange;
    const int rows = (n + xrange - 1) / xrange;
    const int rem = n % xrange;
    xteam[0] = parent[0] + row * xrange * parent[1];
    xteam[1] = parent[1];
    xteam[2] = (row == rows - 1 && rem) ? rem : xrange;
    yteam[0] = parent[0] + col * parent[1];
    yteam[1] = parent[1] * xrange;
    yteam[2] = (rem && col < rem) ? n / xrange + 1 : n / xrange;
}

/* ------------------------------------------------------------------------------------------- */
/* fcollect: reference nvshmemi_fcollect_p2p_allpush_threadgroup,
 *   src/include/non_abi/device/coll/fcollect.cuh:331-344: PE p copies its source into slot p of
 *   every PE's dest.
 * alltoall: reference nvshmemi_alltoall_p2p_allpush_threadgroup,
 *   src/include/non_abi/device/coll/alltoall.cuh:122-143: PE p copies block q of its source into
 *   slot p of PE q's dest.                                                                      */
/* ------------------------------------------------------------------------------------------- */
void oracle_fcollect(int npes, size_t seg, const uint8_t *src, uint8_t *dst) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int q = 0; q < npes; ++q)
        for (int p = 0; p < npes; ++p)
            memcpy(dst + ((size_t)q * npes + p) * seg, src + (size_t)p * seg, seg);
}

void oracle_alltoall(int npes, size_t seg, const uint8_t *src, uint8_t *dst) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int q = 0; q < npes; ++q)
        for (int p = 0; p < npes; ++p)
            memcpy(dst + ((size_t)q * npes + p) * seg, src + ((size_t)p * npes + q) * seg, seg);
}

/* ------------------------------------------------------------------------------------------- */
/* allocator model: reference class mspace, src/host/mem/custom_malloc.cpp:74-237.
 * One address-ordered array of blocks {addr, size, used}; first fit walks it from the lowest
 * address, a split leaves the remainder free, free merges with both neighbours.                */
/* ------------------------------------------------------------------------------------------- */
typedef struct { uint64_t addr, size; int used; } oracle_block_t;
struct oracle_space { oracle_block_t *b; size_t n, cap; };

static void space_insert(oracle_space_t *s, size_t at, oracle_block_t blk) {
    if (s->n == s->cap) {
        s->cap = s->cap ? 2 * s->cap : 16;
        s->b = (oracle_block_t *)realloc(s->b, s->cap * sizeof *s->b);
    }
    memmove(s->b + at + 1, s->b + at, (s->n - at) * sizeof *s->b);
    s->b[at] = blk;
    ++s->n;
}
static void space_remove(oracle_space_t *s, size_t at) {
    memmove(s->b + at, s->b + at + 1, (s->n - at - 1) * sizeof *s->b);
    --s->n;
}
static void space_merge_around(oracle_space_t *s, size_t i) {
    if (i + 1 < s->n && !s->b[i + 1].used && s->b[i].addr + s->b[i].size == s->b[i + 1].addr) {
        s->b[i].size += s->b[i + 1].size;
        space_remove(s, i + 1);
    }
    if (i > 0 && !s->b[i - 1].used && s->b[i - 1].addr + s->b[i - 1].size == s->b[i].addr) {
        s->b[i - 1].size += s->b[i].size;
        space_remove(s, i);
    }
}

oracle_space_t *oracle_space_create(uint64_t base, uint64_t capacity) {
    oracle_space_t *s = (oracle_space_t *)calloc(1, sizeof *s);
    const uint64_t skip = (512 - (base & 511)) & 511; /* custom_malloc.cpp:74-80 */
    if (capacity > skip) {
        oracle_block_t blk = {base + skip, capacity - skip, 0};
        space_insert(s, 0, blk);
    }
    return s;
}
void oracle_space_destroy(oracle_space_t *s) { if (s) { free(s->b); free(s); } }

uint64_t oracle_space_alloc(oracle_space_t *s, uint64_t bytes) {
    if (bytes == 0) return 0;                      /* custom_malloc.cpp:133 */
    bytes = (bytes + 511) & ~(uint64_t)511;        /* :134 */
    for (size_t i = 0; i < s->n; ++i) {            /* :135-153 lowest address first */
        if (s->b[i].used || s->b[i].size < bytes) continue;
        const uint64_t rest = s->b[i].size - bytes;
        s->b[i].size = bytes;
        s->b[i].used = 1;
        if (rest) {
            oracle_block_t blk = {s->b[i].addr + bytes, rest, 0};
            space_insert(s, i + 1, blk);
        }
        return s->b[i].addr;
    }
    return 0;
}

uint64_t oracle_space_align(oracle_space_t *s, uint64_t alignment, uint64_t bytes) {
    if (alignment == 0 || (alignment & (alignment - 1)) || alignment % 8) return 0; /* :184 */
    const uint64_t raw = oracle_space_alloc(s, bytes + alignment);                   /* :186-187 */
    if (!raw) return 0;
    const uint64_t ret = (raw + alignment - 1) / alignment * alignment;              /* :189 */
    if (ret != raw) {                                                                /* :190-194 */
        for (size_t i = 0; i < s->n; ++i) {
            if (s->b[i].addr != raw) continue;
            const uint64_t front = ret - raw;
            s->b[i].addr = ret;
            s->b[i].size -= front;
            oracle_block_t blk = {raw, front, 0};
            space_insert(s, i, blk);
            space_merge_around(s, i);
            break;
        }
    }
    return ret;
}

int oracle_space_free(oracle_space_t *s, uint64_t addr) {
    for (size_t i = 0; i < s->n; ++i) {
        if (s->b[i].addr == addr && s->b[i].used) {  /* :158-167 */
            s->b[i].used = 0;
            space_merge_around(s, i);                /* add_free_chunk :96-128 */
            return 0;
        }
    }
    return -1;
}

/* reallocate (custom_malloc.cpp:198-229): the size is rounded like a request; the same rounded size
 * returns the block; a smaller one keeps the front and frees the tail (:202-206); a larger one grows
 * in place when the chunk right behind the block is free and the two together suffice (:208-219),
 * else takes a fresh block by first fit and frees the old one (:221-226; the copy of the contents is
 * the caller's business here, *moved_from names the old block).  NULL (0) when there is no room: the
 * old block stays.
 * One deviation is pinned on purpose.  In the in-place branch the reference returns
 * `size - current_size` bytes at `ptr + size` to the free list (:216-217), not the real remainder
 * `current_size + chunk_size - size`, so the rest of the consumed chunk is lost and the free chunk it
 * creates can cover memory that is no chunk's at all.  The model (and the library) return the real
 * remainder; tests/golden/allocator_traces.json holds a trace whose later steps tell the two apart.
 * An address that is not a live block returns 0 (the reference would create a zero-size entry). */
uint64_t oracle_space_realloc(oracle_space_t *s, uint64_t addr, uint64_t bytes, uint64_t *moved_from) {
    if (moved_from) *moved_from = 0;
    size_t i = 0;
    while (i < s->n && !(s->b[i].addr == addr && s->b[i].used)) ++i;
    if (i == s->n) return 0;
    bytes = (bytes + 511) & ~(uint64_t)511;
    const uint64_t cur = s->b[i].size;
    if (bytes == cur || bytes == 0) return addr;
    if (bytes < cur) {
        s->b[i].size = bytes;
        oracle_block_t tail = {addr + bytes, cur - bytes, 0};
        space_insert(s, i + 1, tail);
        space_merge_around(s, i + 1);
        return addr;
    }
    if (i + 1 < s->n && !s->b[i + 1].used && s->b[i + 1].addr == addr + cur && cur + s->b[i + 1].size >= bytes) {
        const uint64_t rest = cur + s->b[i + 1].size - bytes;
        s->b[i].size = bytes;
        if (rest) {
            s->b[i + 1].addr = addr + bytes;
            s->b[i + 1].size = rest;
        } else {
            space_remove(s, i + 1);
        }
        return addr;
    }
    const uint64_t fresh = oracle_space_alloc(s, bytes);
    if (!fresh) return 0;
    oracle_space_free(s, addr);
    if (moved_from) *moved_from = addr;
    return fresh;
}

uint64_t oracle_space_free_bytes(const oracle_space_t *s) {
    uint64_t t = 0;
    for (size_t i = 0; i < s->n; ++i) if (!s->b[i].used) t += s->b[i].size;
    return t;
}
uint64_t oracle_space_free_chunks(const oracle_space_t *s) {
    uint64_t t = 0;
    for (size_t i = 0; i < s->n; ++i) if (!s->b[i].used) ++t;
    return t;
}

/* ------------------------------------------------------------------------------------------- */
/* MoE token shuffle model (workload of examples/moe_shuffle.cu)                                 */
/* ------------------------------------------------------------------------------------------- */
/* routing: the reference draws experts per token and rejects duplicates within the token
 * (examples/moe_shuffle.cu:498-512, uniform rand()); here the draw is Zipf(s) by inverse CDF. */
void oracle_moe_routing(int32_t *experts, int tokens, int topk, int num_experts, double zipf_s,
                        uint64_t seed, uint64_t pe) {
    double *cdf = (double *)malloc((size_t)num_experts * sizeof(double));
    double total = 0.0;
    for (int k = 1; k <= num_experts; ++k) { total += pow((double)k, -zipf_s); cdf[k - 1] = total; }
    for (int k = 0; k < num_experts; ++k) cdf[k] /= total;
    cdf[num_experts - 1] = 1.0;
#pragma omp parallel for schedule(static)
    for (int t = 0; t < tokens; ++t) {
        int32_t *row = experts + (size_t)t * topk;
        int have = 0;
        for (uint64_t attempt = 0; have < topk; ++attempt) {
            const uint64_t r = oracle_rand_u64(seed, pe, (uint64_t)t * 65536u + attempt);
            const double u = (double)(r >> 11) * (1.0 / 9007199254740992.0);
            int lo = 0, hi = num_experts - 1; /* first index with cdf >= u */
            while (lo < hi) { const int mid = (lo + hi) / 2; if (cdf[mid] >= u) hi = mid; else lo = mid + 1; }
            int dup = 0;
            for (int j = 0; j < have; ++j) dup |= (row[j] == lo);
            if (!dup) row[have++] = lo;
        }
    }
    free(cdf);
}

/* layout of the receive buffers: rows grouped by (expert, source PE), token order inside a group;
 * the reference obtains the group bases from exchanged per-expert counts and a prefix sum
 * (examples/moe_shuffle.cu:204-234) and the row inside a group from the position in the
 * expert-sorted list (:262-268). */
void oracle_moe_plan(const int32_t *experts, int npes, int tokens, int topk, int num_experts,
                     int64_t *counts, int64_t *seg_base, int32_t *dest_pe, int64_t *dest_row,
                     int64_t *recv_rows) {
    const int epp = num_experts / npes;
    const size_t rows = (size_t)tokens * topk;
    memset(counts, 0, (size_t)npes * num_experts * sizeof(int64_t));
    for (int src = 0; src < npes; ++src)
        for (size_t r = 0; r < rows; ++r) ++counts[(size_t)src * num_experts + experts[src * rows + r]];
    for (int pe = 0; pe < npes; ++pe) {
        int64_t run = 0;
        for (int e = pe * epp; e < (pe + 1) * epp; ++e)
            for (int src = 0; src < npes; ++src) {
                seg_base[(size_t)e * npes + src] = run;
                run += counts[(size_t)src * num_experts + e];
            }
        recv_rows[pe] = run;
    }
    int64_t *next = (int64_t *)malloc((size_t)num_experts * sizeof(int64_t));
    for (int src = 0; src < npes; ++src) {
        for (int e = 0; e < num_experts; ++e) next[e] = seg_base[(size_t)e * npes + src];
        for (size_t r = 0; r < rows; ++r) {
            const int e = experts[src * rows + r];
            dest_pe[src * rows + r] = e / epp;
            dest_row[src * rows + r] = next[e]++;
        }
    }
    free(next);
}

void oracle_moe_dispatch_one(uint8_t *recv_pe, int pe, const uint8_t *send, int npes, int tokens,
                             int topk, size_t row_bytes, const int32_t *dest_pe,
                             const int64_t *dest_row) {
    const size_t rows = (size_t)tokens * topk;
#pragma omp parallel for schedule(static)
    for (size_t g = 0; g < (size_t)npes * rows; ++g) {
        if (dest_pe[g] != pe) continue;
        const size_t src = g / rows, t = (g % rows) / (size_t)topk;
        memcpy(recv_pe + (size_t)dest_row[g] * row_bytes,
               send + (src * (size_t)tokens + t) * row_bytes, row_bytes);
    }
}

void oracle_moe_combine_one(uint8_t *out_src, int src, const uint8_t *const *recv_ptrs, int tokens,
                            int topk, size_t row_bytes, const int32_t *dest_pe,
                            const int64_t *dest_row) {
    const size_t rows = (size_t)tokens * topk;
#pragma omp parallel for schedule(static)
    for (size_t r = 0; r < rows; ++r) {
        const size_t g = (size_t)src * rows + r;
        memcpy(out_src + r * row_bytes, recv_ptrs[dest_pe[g]] + (size_t)dest_row[g] * row_bytes,
               row_bytes);
    }
}
