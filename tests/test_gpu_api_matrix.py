"""GPU parity for the less travelled device API families: typed / sized / strided RMA in all
scopes, scalar p/g of several types, thread-scope put_signal, typed wait / test, sync_all.
Expected values are written out with numpy from the operator definitions (strided forms:
reference src/include/device/nvshmem_defines.h:345-431)."""
import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import note, runtime

pytestmark = pytest.mark.gpu
NPES = 8


def test_api_matrix():
    with runtime(NPES, 16 << 20) as rt:
        perf = rt.perftest()
        a = rt.malloc(8192); b = rt.malloc(8192)
        sig = rt.calloc(4, 8); ints = rt.calloc(8, 4); out = rt.calloc(16, 8)
        A = O.fill_all("bytes", NPES, 8192, 77)
        rt.upload_all(a, A)
        rt.fill(b, 0xEE, 8192)
        note("api_matrix")
        assert perf.nvshmem_perftest_api_matrix(a, b, sig, ints, out, 128, None) == 0
        rt.sync()
        assert all(rt.read_timeout(pe)[0] == 0 for pe in range(NPES)), "a wait gave up"
        B = rt.download_all(b, (8192,), np.uint8)
        OUT = rt.download_all(out, (16,), np.int64)
        SIG = rt.download_all(sig, (4,), np.uint64)
        INTS = rt.download_all(ints, (8,), np.int32)
        for me in range(NPES):
            left, peer = (me - 1) % NPES, (me + 1) % NPES
            want = np.full(8192, 0xEE, np.uint8)
            # 1. contiguous: what my LEFT neighbour put into me, and what I got from my peer
            want[0:64] = A[left, 0:64]                       # double_put, 8 elements
            want[64:74] = A[left, 64:74]                     # put16, 5 elements
            want[128:176] = A[left, 128:176]                 # put128_warp, 3 elements
            want[256:284] = A[peer, 256:284]                 # get32_block, 7 elements
            want[320:333] = A[peer, 320:333]                 # int8_get_nbi_warp, 13 elements
            want[384:402] = A[left, 384:402]                 # ushort_put_nbi_block, 9 elements
            # 2. strided
            w16 = want[512:].view(np.int16); s16 = A[left, 512:].view(np.int16)
            for i in range(10):
                w16[i * 3] = s16[i * 2]                      # int16_iput dst=3 sst=2
            wf = want[1024:].view(np.float32); sf = A[peer, 1024:].view(np.float32)
            for i in range(20):
                wf[i * 2] = sf[i * 3]                        # float_iget_block dst=2 sst=3
            w64 = want[1536:].view(np.int64); s64 = A[left, 1536:].view(np.int64)
            for i in range(6):
                w64[i * 1] = s64[i * 4]                      # int64_iput_warp dst=1 sst=4
            # 3. scalar p from my left neighbour
            want[2048:2052] = np.array([1.5 + left], np.float32).view(np.uint8)
            want[2052] = ord("A") + left
            want[2054:2056] = A[left, 2054:2056]
            want[2056:2064] = np.array([0x1122334455667788 + left], np.uint64).view(np.uint8)
            want[2064:2066] = np.array([-7 - left], np.int16).view(np.uint8)
            # 5. put_signal payloads from my left neighbour
            want[4096:4129] = A[left, 4096:4129]
            want[4160:4172] = A[left, 4160:4172]
            want[4224:4240] = A[left, 4224:4240]
            diff = np.nonzero(B[me] != want)[0]
            assert diff.size == 0, "PE %d: first mismatch at byte %d" % (me, diff[0])
            # 4. scalar g from my peer's a
            o = OUT[me]
            assert o[0] == A[peer, 3072:3080].view(np.int64)[0]
            assert o[1] == A[peer, 3080]
            assert o[2] == A[peer, 3082:3084].view(np.int16)[0]
            assert o[3] == A[peer, 3088:3096].view(np.int64)[0]          # double, compared by bits
            assert o[4] == A[peer, 3096:3098].view(np.uint16)[0]         # half, by bits
            assert o[5] == 7 and o[6] == 11                              # SET 7; ADD 5 + ADD 6
            assert (o[7], o[8], o[9]) == (1, 0, 1)                       # test EQ 103 / LT 5 / all NE 0
            assert o[10] == me * 1000 + NPES and o[11] == me * 100 + NPES
            assert o[12] == 15
            # the set forms of wait / test (any, some, _vector): one bit per check, all must hold
            assert o[13] == 0xFFFF, "set wait/test checks failed: %s" % bin(int(o[13]))
            assert INTS[me, 5] == 77
            assert SIG[me, 0] == 7 and SIG[me, 1] == 11
            assert list(INTS[me, :4]) == [100, 101, 102, 103]
