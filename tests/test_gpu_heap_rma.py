"""GPU parity: symmetric heap, address translation, put/get in the three scopes (a1-a4).
Everything goes through the C ABI; results are compared byte for byte with the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import note, runtime
from nvshmem_amd import hip

pytestmark = pytest.mark.gpu

NPES = 8


@pytest.fixture(scope="module")
def rt():
    with runtime(NPES, 1 << 30) as r:
        yield r


# ---------------------------------------------------------------------------------------------
# heap and nvshmem_ptr
# ---------------------------------------------------------------------------------------------
def test_identity_and_versions(rt):
    assert rt.lib.nvshmem_n_pes() == NPES and rt.lib.nvshmem_my_pe() == 0
    assert rt.lib.nvshmem_team_n_pes(N.TEAM_WORLD) == NPES
    assert rt.lib.nvshmemx_init_status() == 2      # NVSHMEM_STATUS_IS_INITIALIZED
    assert rt.lib.nvshmemx_amd_init(4, 1 << 20) != 0   # second init is refused
    import ctypes as C
    provided = C.c_int32(-1)
    assert rt.lib.nvshmem_init_thread(3, C.byref(provided)) == 0 and provided.value == 2   # SERIALIZED
    assert rt.lib.nvshmem_n_pes() == NPES              # init on a live runtime changes nothing
    provided.value = -1
    rt.lib.nvshmem_query_thread(C.byref(provided))
    assert provided.value == 2
    buf = rt.malloc(64)
    assert rt.lib.nvshmemx_buffer_register(buf, 64) == 0 and rt.lib.nvshmemx_buffer_unregister(buf) == 0
    assert rt.lib.nvshmemx_buffer_register(None, 64) != 0
    rt.free(buf)


def test_pe_identity_follows_grid_z(rt):
    """The one rule that makes a block a PE: a grid whose z extent equals the PE count is a PE grid (block z
    acts as PE z); a kernel launched with any other z extent acts as PE 0 whatever its block index, so a
    kernel that is not meant as a PE kernel must not use z == npes while it calls the device API."""
    perf = rt.perftest()
    out = rt.malloc(128 * 4)       # plain device memory for this kernel: PE 0's copy, used untranslated
    for grid_z in (NPES, 1, 3, NPES - 1, NPES + 1, 2 * NPES):
        note("pe identity, grid z", grid_z)
        rt.fill(out, 0xFF, 128 * 4)
        assert perf.nvshmem_perftest_pe_identity(out, grid_z, None) == 0
        rt.sync()
        got = rt.download(out, 0, (128,), np.int32)
        want = np.arange(grid_z) if grid_z == NPES else np.zeros(grid_z, dtype=np.int32)
        assert np.array_equal(got[:grid_z], want), (grid_z, got[:grid_z])
        assert np.all(got[64:64 + grid_z] == NPES)
        assert np.all(got[grid_z:64] == -1)
    assert perf.nvshmem_perftest_pe_identity(out, 0, None) != 0
    rt.free(out)


def test_malloc_ptr_translation_matches_closed_form(rt):
    a = rt.malloc(1000)
    b = rt.malloc(1)
    assert a % 512 == 0 and b == a + 1024          # 512-byte granules, first fit
    heap_size = rt.ptr(a, 1) - rt.ptr(a, 0)
    # slices are 16 MiB-aligned and no larger than asked for beyond that (no rounding to a power of two)
    assert (1 << 30) <= heap_size <= (1 << 30) + (16 << 20) and heap_size % (16 << 20) == 0
    assert rt.ptr(a, 0) == a                       # canonical address is PE 0's copy
    L = O.lib()
    for pe in range(NPES):
        # closed form of the oracle, written relative to the object (the heap base cancels)
        assert rt.ptr(a + 17, pe) == L.oracle_ptr(a, heap_size, NPES, a + 17, pe)
        assert rt.ptr(a + 17, pe) == a + 17 + pe * heap_size
        assert rt.ptr(rt.ptr(a, 3) + 5, pe) == a + 5 + pe * heap_size   # any PE's copy is accepted
    assert rt.ptr(a, -1) is None and rt.ptr(a, NPES) is None
    assert rt.ptr(0x1000, 0) is None
    assert rt.ptr(a + NPES * heap_size, 0) is None  # past the last slice
    rt.free(a)
    c = rt.malloc(512)
    assert c == a                                  # lowest-address first fit reuses the hole
    rt.free(b); rt.free(c)


def test_zero_size_null_and_calloc_zeroes_every_pe(rt):
    assert rt.lib.nvshmem_malloc(0) is None
    assert rt.lib.nvshmem_calloc(0, 8) is None
    assert rt.lib.nvshmem_align(64, 0) is None
    rt.lib.nvshmem_free(None)                      # no-op
    n = 3000
    dirty = rt.malloc(n)
    rt.fill(dirty, 0xAB, n)
    rt.free(dirty)
    z = rt.calloc(n, 1)
    assert z == dirty
    assert (rt.download_all(z, (n,), np.uint8) == 0).all()
    rt.free(z)
    al = rt.lib.nvshmem_align(1 << 16, 100)
    assert al % (1 << 16) == 0
    assert rt.lib.nvshmem_align(24, 100) is None   # not a power of two
    rt.free(al)


def test_heap_exhaustion_returns_null_with_hint(rt):
    assert rt.lib.nvshmem_malloc(1 << 40) is None
    assert b"NVSHMEM_SYMMETRIC_SIZE" in rt.lib.nvshmemx_amd_last_error()
    rt.lib.nvshmem_free(C.c_void_p(0x12345000))     # not a live block: reported, not fatal
    assert b"not a live symmetric allocation" in rt.lib.nvshmemx_amd_last_error()


# ---------------------------------------------------------------------------------------------
# device-initiated put / get
# ---------------------------------------------------------------------------------------------
def _ring(rt, size, blocks, threads, scope, is_get, src_off=0, dst_off=0, seed=2):
    """One ring exchange; returns (got, expected) as [npes, size] uint8 plus guard checks."""
    perf = rt.perftest()
    pad = 64
    src = rt.malloc(size + 2 * pad)
    dst = rt.malloc(size + 2 * pad)
    data = O.fill_all("bytes", NPES, max(size, 1), seed)[:, :size]
    rt.fill(src, 0x11, size + 2 * pad)
    rt.fill(dst, 0xEE, size + 2 * pad)
    rt.upload_all(src, data, pad + src_off)
    note("ring_rma size=%d blocks=%d threads=%d scope=%d get=%d soff=%d doff=%d"
         % (size, blocks, threads, scope, is_get, src_off, dst_off))
    rc = perf.nvshmem_perftest_ring_rma(dst + pad + dst_off, src + pad + src_off, size, blocks,
                                        threads, scope, is_get, 1, None)
    assert rc == 0
    rt.sync()
    whole = rt.download_all(dst, (size + 2 * pad,), np.uint8)
    rt.free(src); rt.free(dst)
    lo, hi = pad + dst_off, pad + dst_off + size
    assert (whole[:, :lo] == 0xEE).all() and (whole[:, hi:] == 0xEE).all(), "wrote outside the range"
    want = O.ring_get(data) if is_get else O.ring_put(data)
    return whole[:, lo:hi], want


@pytest.mark.parametrize("is_get", [0, 1])
@pytest.mark.parametrize("blocks", [1, 4, 16])
def test_ring_put_get_block_sizes_8B_to_4MiB(rt, blocks, is_get):
    for p in range(3, 23):
        got, want = _ring(rt, 1 << p, blocks, 256, N.SCOPE_BLOCK, is_get)
        assert np.array_equal(got, want), "size 2^%d" % p


# 96 and 160 threads: the block's last wavefront has 32 lanes only
@pytest.mark.parametrize("scope,threads", [(N.SCOPE_THREAD, 64), (N.SCOPE_WARP, 256), (N.SCOPE_BLOCK, 1024),
                                           (N.SCOPE_WARP, 96), (N.SCOPE_WARP, 160), (N.SCOPE_BLOCK, 96)])
def test_ring_put_get_scopes_ragged_sizes(rt, scope, threads):
    for size in (0, 1, 7, 100, 1000, 4097, 65536 + 13, (1 << 20) + 5):
        for is_get in (0, 1):
            got, want = _ring(rt, size, 3, threads, scope, is_get)
            assert np.array_equal(got, want), (size, is_get)


def test_copy_engine_all_mutual_alignments(rt):
    # every source offset mod 16 against a spread of destination offsets, short lengths around the
    # vector width: exercises head, unaligned body loads and tail
    for soff in range(16):
        for doff in (0, 1, 3, 4, 8, 15):
            for size in (1, 15, 16, 17, 31, 64, 255, 300):
                got, want = _ring(rt, size, 1, 64, N.SCOPE_BLOCK, 0, soff, doff, seed=soff * 16 + doff)
                assert np.array_equal(got, want), (soff, doff, size)
    for soff, doff in ((1, 0), (0, 7), (5, 9), (8, 8), (13, 13)):
        for is_get in (0, 1):
            got, want = _ring(rt, 70000 + soff, 4, 256, N.SCOPE_BLOCK, is_get, soff, doff)
            assert np.array_equal(got, want), (soff, doff, is_get)


@pytest.mark.parametrize("is_get", [0, 1])
def test_ring_put_get_256MiB_16_blocks(rt, is_get):
    # the largest message of the sweep: 256 MiB per PE, 16 blocks per PE
    size = 1 << 28
    perf = rt.perftest()
    src = rt.malloc(size); dst = rt.malloc(size)
    data = O.fill_all("bytes", NPES, size, 2)
    rt.upload_all(src, data)
    rt.fill(dst, 0, size)
    note("ring_rma 256MiB get=%d" % is_get)
    assert perf.nvshmem_perftest_ring_rma(dst, src, size, 16, 1024, N.SCOPE_BLOCK, is_get, 1, None) == 0
    rt.sync()
    for pe in range(NPES):
        got = rt.download(dst, pe, (size,), np.uint8)
        want = data[(pe + 1) % NPES] if is_get else data[(pe - 1) % NPES]
        assert np.array_equal(got, want), pe
    rt.free(src); rt.free(dst)


def _sampled_equal(rt, dst, pe, want, size, size_max):
    """Compares windows of the destination instead of all of it: both ends, every slice boundary of a
    16-block launch, and the bytes behind the message, which must still be zero."""
    edges = sorted(set([0, size] + [size // 16 * b for b in range(1, 16)] + [size // 4 * b for b in range(1, 4)]))
    for e in edges:
        lo, hi = max(0, e - (1 << 16)), min(size, e + (1 << 16))
        if hi > lo:
            got = rt.download(dst, pe, (hi - lo,), np.uint8, lo)
            if not np.array_equal(got, want[lo:hi]):
                return False
    tail = min(4096, size_max - size)
    return tail == 0 or bool((rt.download(dst, pe, (tail,), np.uint8, size) == 0).all())


def test_ring_put_get_upper_half_of_the_sweep_every_block_count_and_direction(rt):
    # config 2's sizes from 8 MiB to 256 MiB, each at 1 / 4 / 16 blocks of 1024 threads, put and get:
    # one PE compared in full (it changes from case to case), the others on sampled windows
    perf = rt.perftest()
    size_max = 1 << 28
    src = rt.malloc(size_max); dst = rt.malloc(size_max)
    data = O.fill_all("bytes", NPES, size_max, 3)
    rt.upload_all(src, data)
    case = 0
    for p in range(23, 29):
        for blocks in (1, 4, 16):
            for is_get in (0, 1):
                size = 1 << p
                rt.fill(dst, 0, size_max)
                note("ring_rma size=%d blocks=%d get=%d" % (size, blocks, is_get))
                assert perf.nvshmem_perftest_ring_rma(dst, src, size, blocks, 1024, N.SCOPE_BLOCK, is_get, 1, None) == 0
                rt.sync()
                full = case % NPES
                case += 1
                for pe in range(NPES):
                    want = data[(pe + 1) % NPES] if is_get else data[(pe - 1) % NPES]
                    if pe == full:
                        got = rt.download(dst, pe, (size,), np.uint8)
                        assert np.array_equal(got, want[:size]), (size, blocks, is_get, pe)
                    assert _sampled_equal(rt, dst, pe, want, size, size_max), (size, blocks, is_get, pe)
    rt.free(src); rt.free(dst)


def test_ring_put_get_large_messages_other_scopes_and_the_gpu_filling_shape(rt):
    # warp and thread scope at 64 MiB and more, a ragged 128 MiB + 12345, and the launch shape with one
    # wavefront per KiB at 256 MiB
    perf = rt.perftest()
    size_max = 1 << 28
    src = rt.malloc(size_max); dst = rt.malloc(size_max)
    data = O.fill_all("bytes", NPES, size_max, 4)
    rt.upload_all(src, data)
    cases = [(1 << 26, 16, 256, N.SCOPE_WARP, 0), (1 << 27, 64, 512, N.SCOPE_WARP, 1),
             ((1 << 26) + 77, 256, 256, N.SCOPE_THREAD, 0), (1 << 26, 1024, 64, N.SCOPE_THREAD, 1),
             (size_max, size_max >> 10, 64, N.SCOPE_BLOCK, 0), (size_max, size_max >> 10, 64, N.SCOPE_BLOCK, 1),
             ((1 << 27) + 12345, 1 << 17, 64, N.SCOPE_BLOCK, 0), ((1 << 27) + 12345, 4, 1024, N.SCOPE_BLOCK, 1)]
    for size, blocks, threads, scope, is_get in cases:
        rt.fill(dst, 0, size_max)
        note("ring_rma size=%d blocks=%d threads=%d scope=%d get=%d" % (size, blocks, threads, scope, is_get))
        assert perf.nvshmem_perftest_ring_rma(dst, src, size, blocks, threads, scope, is_get, 1, None) == 0
        rt.sync()
        for pe in (0, 3, NPES - 1):
            got = rt.download(dst, pe, (min(size + 4096, size_max),), np.uint8)
            want = data[(pe + 1) % NPES] if is_get else data[(pe - 1) % NPES]
            assert np.array_equal(got[:size], want[:size]), (size, blocks, pe)
            assert (got[size:] == 0).all(), (size, blocks, pe)
    rt.free(src); rt.free(dst)


@pytest.mark.parametrize("elem", [1, 2, 4, 8])
def test_element_wise_p_g_store_and_atomic_add(rt, elem):
    """One element per thread and call (the reference's shmem_p_bw / g_bw / st_bw / atomic_bw shape):
    the ring shift of the oracle for p, g and the plain store; element-wise wrapping sums for add."""
    perf = rt.perftest()
    kinds = [(0, "p"), (1, "g"), (2, "st")] + ([(3, "add")] if elem >= 4 else [])
    for nelems, blocks, threads in ((1, 1, 64), (1000, 3, 64), (70001, 16, 256), (1 << 18, 64, 1024)):
        size = nelems * elem
        src = rt.malloc(size + 64); dst = rt.malloc(size + 64)
        data = O.fill_all("bytes", NPES, size, 20 + elem)[:, :size]
        start = O.fill_all("bytes", NPES, size + 64, 30 + elem)[:, :size + 64]
        rt.upload_all(src, data)
        for what, name in kinds:
            rt.upload_all(dst, start)
            note("element_bw %s elem=%d nelems=%d blocks=%d threads=%d" % (name, elem, nelems, blocks, threads))
            assert perf.nvshmem_perftest_element_bw(what, elem, dst, src, nelems, blocks, threads, None) == 0
            rt.sync()
            whole = rt.download_all(dst, (size + 64,), np.uint8)
            assert np.array_equal(whole[:, size:], start[:, size:]), "wrote past the range"
            if name == "add":
                ty = np.uint32 if elem == 4 else np.uint64
                want = (start[:, :size].copy().view(ty) + O.ring_put(data).copy().view(ty)).view(np.uint8)
            else:
                want = O.ring_get(data) if name == "g" else O.ring_put(data)
            assert np.array_equal(whole[:, :size], want), (name, nelems)
        rt.free(src); rt.free(dst)
    a = rt.malloc(64)
    assert perf.nvshmem_perftest_element_bw(3, 2, a, a, 4, 1, 64, None) != 0      # no 2-byte atomics
    assert perf.nvshmem_perftest_element_bw(0, 8, a + 4, a, 4, 1, 64, None) != 0  # misaligned for the type
    assert perf.nvshmem_perftest_element_bw(0, 3, a, a, 4, 1, 64, None) != 0
    rt.free(a)


def test_ring_rejects_ranges_outside_the_heap(rt):
    perf = rt.perftest()
    a = rt.malloc(4096)
    assert perf.nvshmem_perftest_ring_rma(a, a + 2048, 1 << 31, 1, 64, 2, 0, 1, None) != 0
    assert perf.nvshmem_perftest_ring_rma(0x1000, a, 16, 1, 64, 2, 0, 1, None) != 0
    assert perf.nvshmem_perftest_ring_rma(a, a, 16, 1, 2048, 2, 0, 1, None) != 0
    rt.free(a)


# ---------------------------------------------------------------------------------------------
# host-initiated RMA and typed wrappers
# ---------------------------------------------------------------------------------------------
def test_host_putmem_getmem_and_typed_forms(rt):
    n = 100003
    a = rt.malloc(n * 8); b = rt.malloc(n * 8)
    data = O.fill_all("u64", NPES, n, 12)
    rt.upload_all(a, data)
    rt.fill(b, 0, n * 8)
    note("host putmem/getmem")
    rt.lib.nvshmem_putmem(b, a, n * 8, 5)                  # PE 0's a -> PE 5's b
    assert np.array_equal(rt.download(b, 5, (n,), np.uint64), data[0])
    rt.lib.nvshmem_getmem(b, a, n * 8, 3)                  # PE 3's a -> PE 0's b
    assert np.array_equal(rt.download(b, 0, (n,), np.uint64), data[3])
    # a source that names another PE's copy explicitly is used as it is
    rt.lib.nvshmem_putmem(b, rt.ptr(a, 6), n * 8, 2)
    assert np.array_equal(rt.download(b, 2, (n,), np.uint64), data[6])
    put = rt.lib.nvshmem_double_put
    put.restype, put.argtypes = None, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    put(b, a, n, 7)
    assert np.array_equal(rt.download(b, 7, (n,), np.uint64), data[0])
    s = hip.Stream()
    get = rt.lib.nvshmemx_int16_get_on_stream
    get.restype, get.argtypes = None, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
    get(b, a, 4 * n, 4, s.ptr)
    s.synchronize()
    assert np.array_equal(rt.download(b, 0, (n,), np.uint64), data[4])
    # bad PE / non-symmetric target are reported, nothing is copied
    rt.lib.nvshmem_putmem(b, a, 8, 99)
    assert b"pe 99" in rt.lib.nvshmemx_amd_last_error()
    rt.lib.nvshmem_putmem(0x2000, a, 8, 1)
    assert b"not a symmetric address" in rt.lib.nvshmemx_amd_last_error()
    s.destroy()
    rt.free(a); rt.free(b)
