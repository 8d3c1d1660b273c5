"""GPU parity for single calls that move more than 2^32 bytes (and, for 1-byte elements, more than 2^32
elements).  The reference's loops carry 32-bit indices in several places on this path
(coll/reduce.cuh:118-121 `int i`, coll/alltoall.cuh:127-137 `int` offsets, coll/fcollect.cuh:374 `int
dest_offset`); here every index is 64-bit, and these cases would wrap if one were not."""
import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import note, runtime

pytestmark = pytest.mark.gpu

NPES = 2
BIG = (1 << 32) + (3 << 20) + 4096 + 24      # bytes per PE: past 2^32, not a multiple of 1 KiB
SALT = np.uint64(0x9E3779B97F4A7C15)


def _pattern(pe, nwords):
    """Position-dependent 64-bit words, so that a wrapped index lands on different data."""
    x = np.arange(nwords, dtype=np.uint64)
    x *= SALT
    x += np.uint64(0x1234567 * (pe + 1))
    x ^= x >> np.uint64(29)
    return x


@pytest.fixture(scope="module")
def rt():
    with runtime(NPES, 3 * BIG + (64 << 20)) as r:
        yield r


@pytest.fixture(scope="module")
def data():
    return [_pattern(pe, BIG // 8).view(np.uint8) for pe in range(NPES)]


def _equal_in_pieces(rt, sym, pe, want, byte_offset=0):
    """Downloads and compares 512 MiB at a time (bounded host memory)."""
    step = 1 << 29
    for lo in range(0, want.nbytes, step):
        hi = min(want.nbytes, lo + step)
        got = rt.download(sym, pe, (hi - lo,), np.uint8, byte_offset + lo)
        if not np.array_equal(got, want[lo:hi]):
            return False
    return True


def test_put_and_get_of_more_than_4gib_per_call(rt, data):
    perf = rt.perftest()
    src = rt.malloc(BIG); dst = rt.malloc(BIG)
    rt.upload_all(src, data)
    for is_get, blocks, threads, scope in ((0, 16, 1024, N.SCOPE_BLOCK), (1, 4, 1024, N.SCOPE_BLOCK),
                                           (0, 64, 256, N.SCOPE_WARP)):
        rt.fill(dst, 0, BIG)
        note("ring rma of %d bytes per PE, get=%d blocks=%d threads=%d scope=%d" % (BIG, is_get, blocks, threads, scope))
        assert perf.nvshmem_perftest_ring_rma(dst, src, BIG, blocks, threads, scope, is_get, 1, None) == 0
        rt.sync()
        for pe in range(NPES):
            source = (pe + 1) % NPES if is_get else (pe - 1) % NPES
            assert _equal_in_pieces(rt, dst, pe, data[source]), (is_get, blocks, pe)
    rt.free(src); rt.free(dst)


def test_collectives_of_more_than_4gib_per_call(rt, data):
    src = rt.malloc(BIG); dst = rt.malloc(2 * BIG)
    rt.upload_all(src, data)
    # fcollect: every PE's 4 GiB + ... land behind each other; slot 1 starts past 2^32
    note("fcollectmem of %d bytes per PE" % BIG)
    rt.fcollectmem(dst, src, BIG)
    for pe in range(NPES):
        for p in range(NPES):
            assert _equal_in_pieces(rt, dst, pe, data[p], p * BIG), (pe, p)
    # alltoall with blocks of more than 2 GiB (offsets of block 1 exceed a signed 32-bit index)
    seg = BIG // 2 // 8 * 8
    note("alltoallmem with blocks of %d bytes" % seg)
    rt.alltoallmem(dst, src, seg)
    for q in range(NPES):
        for p in range(NPES):
            assert _equal_in_pieces(rt, dst, q, data[p][q * seg:(q + 1) * seg], p * seg), (q, p)
    # broadcast from PE 1
    note("broadcastmem of %d bytes" % BIG)
    rt.fill(dst, 0, BIG)
    rt.broadcastmem(dst, src, BIG, 1)
    assert _equal_in_pieces(rt, dst, 0, data[1])
    # allreduce over more than 2^32 one-byte elements, and over 2^29 + 387 eight-byte ones
    n8 = BIG - 24
    note("uint8 xor reduce of %d elements" % n8)
    rt.reduce("uint8", "xor", dst, src, n8)
    want = data[0][:n8] ^ data[1][:n8]
    assert _equal_in_pieces(rt, dst, 0, want) and _equal_in_pieces(rt, dst, 1, want)
    n64 = BIG // 8
    note("int64 sum reduce of %d elements" % n64)
    rt.reduce("int64", "sum", dst, src, n64)
    want = (data[0].view(np.uint64) + data[1].view(np.uint64)).view(np.uint8)     # wraps, like the kernel
    assert _equal_in_pieces(rt, dst, 1, want)
    # reducescatter: block 1 of every source lies past 2^31 bytes
    half = n64 // 2
    note("int64 xor reducescatter of 2 x %d elements" % half)
    rt.reducescatter("int64", "xor", dst, src, half)
    for q in range(NPES):
        a = data[0].view(np.uint64)[q * half:(q + 1) * half]
        b = data[1].view(np.uint64)[q * half:(q + 1) * half]
        assert _equal_in_pieces(rt, dst, q, (a ^ b).view(np.uint8)), q
    rt.free(src); rt.free(dst)
