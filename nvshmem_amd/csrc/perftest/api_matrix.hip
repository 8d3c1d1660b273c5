// One kernel that walks through the less travelled corners of the device API - typed, sized and
// strided RMA in all scopes, scalar p/g of several types, thread-scope put_signal, typed waits and
// tests, sync_all, quiet/fence - with a layout simple enough to predict on the host.
// The API families are those of the reference's src/include/device/nvshmem_defines.h:80-740 and
// src/include/device/nvshmemx_defines.h:35-451.
#include <hip/hip_runtime.h>

#include "nvshmem_perftest.h"
#include "nvshmemx.h"
#include "perftest_common.hpp"

namespace {

// a, b: 8 KiB symmetric byte buffers; sig: 4 uint64; ints: 8 int32; out: 16 int64 (all symmetric).
// Every PE acts on its right neighbour `peer`; `left` is the PE that acts on this one.
__global__ void api_matrix_kernel(char *a, char *b, uint64_t *sig, int *ints, int64_t *out) {
    const int me = nvshmem_my_pe(), np = nvshmem_n_pes();
    const int peer = (me + 1) % np;
    const bool t0 = threadIdx.x == 0;
    const bool wave0 = threadIdx.x < NVSHMEMI_WARP_SIZE;
    int64_t *my_out = (int64_t *)nvshmem_ptr(out, me);

    // 1. typed and sized contiguous RMA
    if (t0) nvshmem_double_put((double *)b, (const double *)a, 8, peer);            // b@peer[0,64)
    if (t0) nvshmem_put16(b + 64, a + 64, 5, peer);                                // b@peer[64,74)
    if (wave0) nvshmemx_put128_warp(b + 128, a + 128, 3, peer);                    // b@peer[128,176)
    nvshmemx_get32_block(b + 256, a + 256, 7, peer);                               // b@me[256,284)
    if (wave0) nvshmemx_int8_get_nbi_warp((int8_t *)b + 320, (const int8_t *)a + 320, 13, peer);
    nvshmemx_ushort_put_nbi_block((unsigned short *)(b + 384), (const unsigned short *)(a + 384), 9, peer);
    // 2. strided RMA: element i of the source at stride sst -> element i*dst of the destination
    if (t0) nvshmem_int16_iput((int16_t *)(b + 512), (const int16_t *)(a + 512), 3, 2, 10, peer);
    nvshmemx_float_iget_block((float *)(b + 1024), (const float *)(a + 1024), 2, 3, 20, peer);
    if (wave0) nvshmemx_int64_iput_warp((int64_t *)(b + 1536), (const int64_t *)(a + 1536), 1, 4, 6, peer);
    // 3. scalar p of several types
    if (t0) {
        nvshmem_float_p((float *)(b + 2048), 1.5f + (float)me, peer);
        nvshmem_char_p(b + 2052, (char)('A' + me), peer);
        nvshmem_bfloat16_p((nvshmem_bfloat16_t *)(b + 2054), *(const nvshmem_bfloat16_t *)nvshmem_ptr(a + 2054, me), peer);
        nvshmem_uint64_p((uint64_t *)(b + 2056), 0x1122334455667788ull + (uint64_t)me, peer);
        nvshmem_short_p((short *)(b + 2064), (short)(-7 - me), peer);
    }
    nvshmemx_barrier_all_block();
    // 4. scalar g of several types from the peer's `a`
    if (t0) {
        my_out[0] = nvshmem_int64_g((const int64_t *)(a + 3072), peer);
        my_out[1] = (int64_t)nvshmem_uint8_g((const uint8_t *)(a + 3080), peer);
        my_out[2] = (int64_t)nvshmem_short_g((const short *)(a + 3082), peer);
        const double d = nvshmem_double_g((const double *)(a + 3088), peer);
        __builtin_memcpy(&my_out[3], &d, 8);
        const nvshmem_half_t h = nvshmem_half_g((const nvshmem_half_t *)(a + 3096), peer);
        uint16_t hb;
        __builtin_memcpy(&hb, &h, 2);
        my_out[4] = hb;
    }
    // 5. thread-scope put with signal, typed waits and tests
    if (t0) {
        nvshmem_putmem_signal(b + 4096, a + 4096, 33, sig, 7, NVSHMEM_SIGNAL_SET, peer);
        nvshmem_uint64_wait_until(sig, NVSHMEM_CMP_EQ, 7);          // my left neighbour's signal
        my_out[5] = (int64_t)nvshmem_signal_fetch(sig);
        nvshmem_int32_put_signal((int32_t *)(b + 4160), (const int32_t *)(a + 4160), 3, sig + 1, 5,
                                 NVSHMEM_SIGNAL_ADD, peer);
        nvshmem_put64_signal_nbi(b + 4224, a + 4224, 2, sig + 1, 6, NVSHMEM_SIGNAL_ADD, peer);
        my_out[6] = (int64_t)nvshmem_signal_wait_until(sig + 1, NVSHMEM_CMP_GE, 11);
        // typed wait / test on an int array the left neighbour fills with p
        for (int k = 0; k < 4; ++k) nvshmem_int_p(ints + k, 100 + k, peer);
        const int skip[4] = {0, 1, 0, 0};                            // element 1 is not waited for
        nvshmem_int_wait_until_all(ints, 4, skip, NVSHMEM_CMP_GE, 100);
        my_out[7] = nvshmem_int_test(ints + 3, NVSHMEM_CMP_EQ, 103);
        my_out[8] = nvshmem_int_test(ints + 3, NVSHMEM_CMP_LT, 5);
        my_out[9] = nvshmem_int_test_all(ints, 4, skip, NVSHMEM_CMP_NE, 0);
        nvshmem_int_wait_until(ints + 1, NVSHMEM_CMP_EQ, 101);
        // set forms: ints[0..4) now hold 100..103; the left neighbour also sets ints[5] = 77
        nvshmem_int_p(ints + 5, 77, peer);
        {
            int *mine = (int *)nvshmem_ptr(ints, me);
            size_t idx[8];
            const int skip2[8] = {0, 0, 1, 0, 0, 0, 0, 0};
            const int all_skipped[4] = {1, 1, 1, 1};
            int exact[4] = {100, 101, 102, 103}, wrong[4] = {100, 101, 0, 103}, below[4] = {100, 101, 101, 103};
            unsigned ok = 0;
            ok |= (nvshmem_int_test_any(mine, 4, nullptr, NVSHMEM_CMP_EQ, 102) == 2) << 0;
            ok |= (nvshmem_int_test_any(mine, 4, skip2, NVSHMEM_CMP_GE, 102) == 3) << 1;
            ok |= (nvshmem_int_test_any(mine, 4, nullptr, NVSHMEM_CMP_GT, 1000) == SIZE_MAX) << 2;
            ok |= (nvshmem_int_test_some(mine, 4, idx, nullptr, NVSHMEM_CMP_GE, 101) == 3 && idx[0] == 1 &&
                   idx[1] == 2 && idx[2] == 3) << 3;
            ok |= (nvshmem_int_test_some(mine, 4, idx, skip2, NVSHMEM_CMP_LT, 100) == 0) << 4;
            ok |= (nvshmem_int_test_all_vector(mine, 4, nullptr, NVSHMEM_CMP_EQ, exact) == 1) << 5;
            ok |= (nvshmem_int_test_all_vector(mine, 4, nullptr, NVSHMEM_CMP_EQ, wrong) == 0) << 6;
            ok |= (nvshmem_int_test_all_vector(mine, 4, skip2, NVSHMEM_CMP_EQ, wrong) == 1) << 7;
            ok |= (nvshmem_int_test_any_vector(mine, 4, nullptr, NVSHMEM_CMP_GT, below) == 2) << 8;
            ok |= (nvshmem_int_test_some_vector(mine, 4, idx, nullptr, NVSHMEM_CMP_NE, wrong) == 1 && idx[0] == 2) << 9;
            // waits on ints[4..8): only ints[5] ever changes
            ok |= (nvshmem_int_wait_until_any(mine + 4, 4, nullptr, NVSHMEM_CMP_NE, 0) == 1) << 10;
            ok |= (nvshmem_int_wait_until_some(mine + 4, 4, idx, nullptr, NVSHMEM_CMP_EQ, 77) == 1 && idx[0] == 1) << 11;
            ok |= (nvshmem_int_wait_until_any(mine, 4, all_skipped, NVSHMEM_CMP_EQ, 5) == SIZE_MAX) << 12;
            nvshmem_int_wait_until_all_vector(mine, 4, nullptr, NVSHMEM_CMP_EQ, exact);
            ok |= (nvshmem_int_wait_until_any_vector(mine, 4, nullptr, NVSHMEM_CMP_GT, below) == 2) << 13;
            ok |= (nvshmem_int_wait_until_some_vector(mine, 4, idx, nullptr, NVSHMEM_CMP_GE, exact) == 4 && idx[3] == 3) << 14;
            ok |= (nvshmem_uint64_test_any(sig, 2, nullptr, NVSHMEM_CMP_EQ, 11) == 1) << 15;
            my_out[13] = ok;
        }
        nvshmem_quiet();
        nvshmem_fence();
        my_out[10] = me * 1000 + np;
    }
    nvshmemx_quiet_block();
    nvshmemx_sync_all_block();
    if (wave0) nvshmemx_sync_all_warp();
    if (t0) {
        nvshmem_sync_all();
        my_out[11] = nvshmem_team_my_pe(NVSHMEM_TEAM_WORLD) * 100 + nvshmem_team_n_pes(NVSHMEM_TEAM_WORLD);
        // nvshmem_ptr: valid PE, invalid PE, address outside the heap
        my_out[12] = (nvshmem_ptr(a, peer) != nullptr) + 2 * (nvshmem_ptr(a, np) == nullptr) +
                     4 * (nvshmem_ptr(&my_out, 0) == nullptr) +
                     8 * ((char *)nvshmem_ptr(a + 5, peer) - (char *)nvshmem_ptr(a, peer) == 5);
    }
}

}  // namespace

extern "C" int nvshmem_perftest_api_matrix(void *a, void *b, uint64_t *sig, int *ints, int64_t *out,
                                           int threads, void *stream) {
    if (!perftest::ready() || !perftest::check_launch(1, threads) || threads < NVSHMEMI_WARP_SIZE ||
        !perftest::check_range(a, 8192) || !perftest::check_range(b, 8192) ||
        !perftest::check_range(sig, 4 * sizeof(uint64_t)) || !perftest::check_range(ints, 8 * sizeof(int)) ||
        !perftest::check_range(out, 16 * sizeof(int64_t)))
        return NVSHMEMX_ERROR_INVALID_VALUE;
    char *pa = (char *)a, *pb = (char *)b;
    void *args[] = {&pa, &pb, &sig, &ints, &out};
    return nvshmemx_collective_launch((const void *)api_matrix_kernel, dim3(1), dim3(threads), args, 0,
                                      (hipStream_t)stream);
}
