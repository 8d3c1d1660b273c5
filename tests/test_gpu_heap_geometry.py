"""Heap geometry: the distance between PE slices is the requested size rounded up to 16 MiB (2 MiB for
small heaps), not to a power of two (a2: PE -> address translation on such a heap)."""
import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import note, runtime

pytestmark = pytest.mark.gpu


def test_heap_whose_size_is_no_power_of_two():
    """NVSHMEM_SYMMETRIC_SIZE = 96 MiB + 12345 bytes on 5 PEs: the slices are 112 MiB apart (no rounding to
    128 MiB), translation, ring put / get and an allreduce work as on any other heap."""
    npes, want_size = 5, (96 << 20) + 12345
    with runtime(npes, want_size) as r:
        perf = r.perftest()
        a = r.malloc(1 << 20)
        stride = r.ptr(a, 1) - r.ptr(a, 0)
        assert stride == 112 << 20
        assert r.ptr(r.ptr(a, 4) + 5, 2) == a + 5 + 2 * stride        # any PE's copy names the object
        assert r.ptr(a + npes * stride, 0) is None
        r.free(a)
        size = (40 << 20) + 3
        src = r.malloc(size); dst = r.malloc(size)
        data = O.fill_all("bytes", npes, size, 9)
        r.upload_all(src, data)
        for is_get, blocks, threads in ((0, 16, 1024), (1, 4, 256)):
            r.fill(dst, 0, size)
            note("non-power-of-two heap: ring_rma get=%d" % is_get)
            assert perf.nvshmem_perftest_ring_rma(dst, src, size, blocks, threads, N.SCOPE_BLOCK, is_get, 1, None) == 0
            r.sync()
            want = O.ring_get(data) if is_get else O.ring_put(data)
            assert np.array_equal(r.download_all(dst, (size,), np.uint8), want)
        n = 1000003
        ints = O.fill_all("i32", npes, n, 1)
        r.upload_all(src, ints)
        r.reduce("int32", "sum", dst, src, n)
        r.sync()
        want = O.reduce("i32", "sum", ints)
        assert all(np.array_equal(r.download(dst, pe, (n,), np.int32), want) for pe in range(npes))
        # the usable part of a slice ends where the runtime's own words begin
        r.lib.nvshmem_putmem(src, src, stride, 1)              # a range that runs into the runtime's words
        assert b"leaves the PE's heap slice" in r.lib.nvshmemx_amd_last_error()
        r.free(src); r.free(dst)
