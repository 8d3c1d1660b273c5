"""GPU parity for team sizes other than the headline 8 / 16: 1, 2, 3, 5 (not a power of two),
32 and 64 (the reduce kernel then gives a PE fewer than 64 lanes)."""
import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import bits_equal, note, runtime

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("npes", [1, 2, 3, 5, 32, 64])
def test_collectives_and_rma_for_team_size(npes):
    rng = np.random.default_rng(npes)
    with runtime(npes, 16 << 20) as rt:
        perf = rt.perftest()
        assert rt.lib.nvshmem_n_pes() == npes
        n = 5003
        src = rt.malloc(npes * n * 8 + 64); dst = rt.malloc(npes * n * 8 + 64)
        # host-launched reduce: fp32 sum (order-sensitive), bf16 max, int64 xor, in place too
        f = (rng.standard_normal((npes, n)) * 10.0 ** rng.integers(-3, 4, (npes, n))).astype(np.float32)
        rt.upload_all(src, f)
        note("npes=%d float sum" % npes)
        rt.reduce("float", "sum", dst, src, n)
        want = O.reduce("f32", "sum", f)
        for pe in {0, npes // 2, npes - 1}:
            assert bits_equal(rt.download(dst, pe, (n,), np.float32), want), pe
        rt.reduce("float", "sum", src, src, n)
        assert bits_equal(rt.download(src, npes - 1, (n,), np.float32), want)
        b = (rng.standard_normal((npes, n)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        rt.upload_all(src, b)
        rt.reduce("bfloat16", "max", dst, src, n)
        assert bits_equal(rt.download(dst, 0, (n,), np.uint16), O.reduce("bf16", "max", b))
        x = rng.integers(-2**63, 2**63 - 1, (npes, n), dtype=np.int64)
        rt.upload_all(src, x)
        rt.reduce("int64", "xor", dst, src, n)
        assert np.array_equal(rt.download(dst, npes - 1, (n,), np.int64), O.reduce("i64", "xor", x))
        # fcollect / alltoall with a ragged block size
        seg = 1237
        data = rng.integers(0, 256, (npes, npes * seg), dtype=np.uint8)
        rt.upload_all(src, data)
        note("npes=%d alltoall/fcollect" % npes)
        rt.alltoallmem(dst, src, seg)
        assert np.array_equal(rt.download_all(dst, (npes * seg,), np.uint8), O.alltoall(data))
        rt.fcollectmem(dst, src, seg)
        assert np.array_equal(rt.download_all(dst, (npes * seg,), np.uint8), O.fcollect(data[:, :seg]))
        # device-initiated ring put and the in-kernel barrier / reduce / alltoall
        note("npes=%d device ring put" % npes)
        assert perf.nvshmem_perftest_ring_rma(dst, src, 70001, 2, 256, N.SCOPE_BLOCK, 0, 1, None) == 0
        rt.sync()
        got = rt.download_all(dst, (70001,), np.uint8)
        raw = rt.download_all(src, (70001,), np.uint8)
        assert np.array_equal(got, O.ring_put(raw))
        counter = rt.calloc(1, 8); errors = rt.calloc(1, 8)
        note("npes=%d device barrier" % npes)
        assert perf.nvshmem_perftest_device_barrier(counter, errors, 50, N.SCOPE_BLOCK, 128, None) == 0
        rt.sync()
        assert not rt.download_all(errors, (1,), np.uint64).any()
        ints = rng.integers(-2**20, 2**20, (npes, n), dtype=np.int32)
        rt.upload_all(src, ints)
        note("npes=%d device reduce" % npes)
        assert perf.nvshmem_perftest_device_reduce(N.DTYPES["i32"], N.OPS["sum"], dst, src, n,
                                                   N.SCOPE_BLOCK, 256, None) == 0
        rt.sync()
        assert np.array_equal(rt.download(dst, npes - 1, (n,), np.int32), O.reduce("i32", "sum", ints))
        rt.upload_all(src, data)
        assert perf.nvshmem_perftest_device_alltoall(dst, src, seg, N.SCOPE_WARP, 64, None) == 0
        rt.sync()
        assert np.array_equal(rt.download_all(dst, (npes * seg,), np.uint8), O.alltoall(data))
        # the packet paths of the in-kernel collectives (a few bytes per member), twice each
        for rep in range(2):
            small = rng.integers(-2**20, 2**20, (npes, max(npes * 4, 8)), dtype=np.int32)
            raw = small.view(np.uint8)
            rt.upload_all(src, small)
            note("npes=%d small in-kernel collectives rep=%d" % (npes, rep))
            assert perf.nvshmem_perftest_device_reduce(N.DTYPES["i32"], N.OPS["sum"], dst, src, 4,
                                                       N.SCOPE_BLOCK, 256, None) == 0
            rt.sync()
            want = O.reduce("i32", "sum", small[:, :4])
            assert all(np.array_equal(rt.download(dst, pe, (4,), np.int32), want) for pe in range(npes))
            assert perf.nvshmem_perftest_device_reducescatter(N.DTYPES["i32"], N.OPS["sum"], dst, src, 2,
                                                              N.SCOPE_BLOCK, 256, None) == 0
            rt.sync()
            assert np.array_equal(rt.download_all(dst, (2,), np.int32),
                                  O.reducescatter("i32", "sum", np.ascontiguousarray(small[:, :npes * 2])))
            assert perf.nvshmem_perftest_device_fcollect(dst, src, 8, N.SCOPE_WARP, 64, None) == 0
            rt.sync()
            assert np.array_equal(rt.download_all(dst, (npes * 8,), np.uint8), O.fcollect(raw[:, :8]))
            assert perf.nvshmem_perftest_device_alltoall(dst, src, 8, N.SCOPE_BLOCK, 512, None) == 0
            rt.sync()
            assert np.array_equal(rt.download_all(dst, (npes * 8,), np.uint8),
                                  O.alltoall(np.ascontiguousarray(raw[:, :npes * 8])))
            assert perf.nvshmem_perftest_device_broadcast(dst, src, 21, npes - 1, N.SCOPE_THREAD, 64, None) == 0
            rt.sync()
            assert all(np.array_equal(rt.download(dst, pe, (21,), np.uint8), raw[npes - 1, :21]) for pe in range(npes))
        assert all(rt.read_timeout(pe)[0] == 0 for pe in range(npes))


def test_init_rejects_bad_team_sizes():
    lib = N.load()
    assert lib.nvshmemx_amd_init(0, 1 << 20) != 0
    assert lib.nvshmemx_amd_init(65, 1 << 20) != 0
    assert lib.nvshmemx_init_status() == 0


@pytest.mark.parametrize("npes", [1, 2, 3, 16, 24, 32, 33, 64])
def test_broadcast_and_reducescatter_on_other_team_sizes(npes):
    rng = np.random.default_rng(npes)
    n = 2052
    with runtime(npes, 1 << 22) as rt:
        src = rt.malloc(npes * n * 4); dst = rt.malloc(n * 4)
        data = rng.standard_normal((npes, npes * n)).astype(np.float32)
        rt.upload_all(src, data)
        note("npes=%d reducescatter float sum" % npes)
        rt.reducescatter("float", "sum", dst, src, n)
        assert bits_equal(rt.download_all(dst, (n,), np.float32), O.reducescatter("f32", "sum", data))
        idata = rng.integers(-2**31, 2**31 - 1, (npes, npes * n), dtype=np.int32)
        rt.upload_all(src, idata)
        rt.reducescatter("int32", "xor", dst, src, n)
        assert bits_equal(rt.download_all(dst, (n,), np.int32), O.reducescatter("i32", "xor", idata))
        root = npes - 1
        note("npes=%d broadcast root=%d" % (npes, root))
        rt.broadcastmem(dst + 1, src + 3, n * 4 - 7, root)
        got = rt.download_all(dst, (n * 4 - 7,), np.uint8, 1)
        want = idata.view(np.uint8)[root, 3:3 + n * 4 - 7]
        assert all(np.array_equal(got[pe], want) for pe in range(npes))
        # (value, location) maximum of one pair per PE: packets up to 32 PEs, barriers beyond
        pairs = np.stack([rng.integers(0, 3, (npes, 1)).astype(np.float64),
                          np.arange(npes, dtype=np.float64)[:, None]], axis=2)
        rt.upload_all(src, pairs)
        note("npes=%d maxloc" % npes)
        assert rt.perftest().nvshmem_perftest_device_maxloc(N.TEAM_WORLD, dst, src, 1, 3, 128, None, None) == 0
        rt.sync()
        assert bits_equal(rt.download_all(dst, (1, 2), np.float64), O.maxloc_reduce(pairs))
        rt.free(src); rt.free(dst)


@pytest.mark.parametrize("disable,plain", [("1", "0"), ("0", "0"), ("0", "1")])
def test_small_in_kernel_collectives_with_and_without_packets(disable, plain, monkeypatch):
    """NVSHMEM_AMD_DISABLE_LL=1 (read at init) sends every in-kernel collective through its copy and
    barrier path; NVSHMEM_AMD_PLAIN_COLLECTIVE_LAUNCH=1 starts the PE kernels with an ordinary launch
    after the occupancy check.  Results are the same every way."""
    monkeypatch.setenv("NVSHMEM_AMD_DISABLE_LL", disable)
    monkeypatch.setenv("NVSHMEM_AMD_PLAIN_COLLECTIVE_LAUNCH", plain)
    rng = np.random.default_rng(int(disable))
    with runtime(8, 1 << 22) as rt:
        perf = rt.perftest()
        n = 16
        src = rt.malloc(8 * n * 4); dst = rt.malloc(8 * n * 4)
        for rep in range(5):
            data = rng.standard_normal((8, 8 * n)).astype(np.float32)
            rt.upload_all(src, data)
            note("packets disabled=%s rep=%d" % (disable, rep))
            assert perf.nvshmem_perftest_device_reduce(N.DTYPES["f32"], N.OPS["sum"], dst, src, n,
                                                       N.SCOPE_BLOCK, 256, None) == 0
            rt.sync()
            want = O.reduce("f32", "sum", data[:, :n])
            assert all(bits_equal(rt.download(dst, pe, (n,), np.float32), want) for pe in range(8))
            assert perf.nvshmem_perftest_device_reducescatter(N.DTYPES["f32"], N.OPS["sum"], dst, src, n,
                                                              N.SCOPE_WARP, 64, None) == 0
            rt.sync()
            assert bits_equal(rt.download_all(dst, (n,), np.float32), O.reducescatter("f32", "sum", data))
            raw = data.view(np.uint8)
            assert perf.nvshmem_perftest_device_alltoall(dst, src, n * 4, N.SCOPE_BLOCK, 128, None) == 0
            rt.sync()
            assert np.array_equal(rt.download_all(dst, (8 * n * 4,), np.uint8), O.alltoall(raw))
            assert perf.nvshmem_perftest_device_fcollect(dst, src, n * 4, N.SCOPE_BLOCK, 128, None) == 0
            rt.sync()
            assert np.array_equal(rt.download_all(dst, (8 * n * 4,), np.uint8), O.fcollect(raw[:, :n * 4]))
            assert perf.nvshmem_perftest_device_broadcast(dst, src, n * 4, rep % 8, N.SCOPE_THREAD, 64, None) == 0
            rt.sync()
            assert all(np.array_equal(rt.download(dst, pe, (n * 4,), np.uint8), raw[rep % 8, :n * 4]) for pe in range(8))
            pairs = data[:, :2].astype(np.float64).reshape(8, 1, 2)
            rt.upload_all(src, pairs)
            assert perf.nvshmem_perftest_device_maxloc(N.TEAM_WORLD, dst, src, 1, 2, 64, None, None) == 0
            rt.sync()
            assert bits_equal(rt.download_all(dst, (1, 2), np.float64), O.maxloc_reduce(pairs))
        assert rt.read_timeout(0)[0] == 0
        rt.free(src); rt.free(dst)


@pytest.mark.parametrize("npes", [3, 8, 13, 16, 33, 64])
def test_large_source_policy_of_fcollect_and_broadcast(npes, monkeypatch):
    """Sources beyond NVSHMEM_AMD_CACHEABLE_SOURCE_BYTES (read at init) are streamed, and from
    NVSHMEM_AMD_CHUNKED_COPY_BYTES on fcollect / broadcast split the destinations of a piece over several
    wavefronts (two per wavefront, the grid walking a chunk of the message once per pair).  With the
    thresholds at zero every size takes that path: ragged, misaligned messages must come out the same, bytes
    outside the destination untouched."""
    monkeypatch.setenv("NVSHMEM_AMD_CACHEABLE_SOURCE_BYTES", "0")
    monkeypatch.setenv("NVSHMEM_AMD_CHUNKED_COPY_BYTES", "0")
    monkeypatch.setenv("NVSHMEM_AMD_LDS_REDUCE_BYTES", "0")      # 8 and 16 members: the LDS-staged allreduce
    rng = np.random.default_rng(100 + npes)
    with runtime(npes, 1 << 24) as rt:
        cap = 1 << 16
        src = rt.malloc(cap + 64); dst = rt.malloc(npes * cap + 64)
        for nbytes, soff, doff in ((1, 0, 0), (15, 1, 2), (16, 0, 0), (1023, 3, 0), (1024, 0, 16), (4100, 5, 9),
                                   (65536, 0, 0), (40001, 16, 3)):
            data = rng.integers(0, 256, (npes, nbytes), dtype=np.uint8)
            rt.upload_all(src, data, soff)
            rt.fill(dst, 0xCD, npes * cap + 64)
            note("large-source path npes=%d fcollect bytes=%d soff=%d doff=%d" % (npes, nbytes, soff, doff))
            rt.fcollectmem(dst + doff, src + soff, nbytes)
            got = rt.download_all(dst, (npes * nbytes + doff + 16,), np.uint8)
            assert np.array_equal(got[:, doff:doff + npes * nbytes], O.fcollect(data)), (nbytes, soff, doff)
            assert (got[:, :doff] == 0xCD).all() and (got[:, doff + npes * nbytes:] == 0xCD).all()
            root = (nbytes + soff) % npes
            rt.fill(dst, 0xCD, npes * cap + 64)
            note("large-source path npes=%d broadcast bytes=%d root=%d" % (npes, nbytes, root))
            rt.broadcastmem(dst + doff, src + soff, nbytes, root)
            got = rt.download_all(dst, (nbytes + doff + 16,), np.uint8)
            assert np.array_equal(got[:, doff:doff + nbytes], O.broadcast(data, root)), (nbytes, soff, doff)
            assert (got[:, :doff] == 0xCD).all() and (got[:, doff + nbytes:] == 0xCD).all()
        # reductions and alltoall with streamed sources
        n = 3000
        fsrc = rt.malloc(npes * n * 4); fdst = rt.malloc(npes * n * 4)
        fdata = rng.standard_normal((npes, npes * n)).astype(np.float32)
        rt.upload_all(fsrc, fdata)
        rt.reducescatter("float", "sum", fdst, fsrc, n)
        assert bits_equal(rt.download_all(fdst, (n,), np.float32), O.reducescatter("f32", "sum", fdata))
        rt.reduce("float", "sum", fdst, fsrc, n)
        want = O.reduce("f32", "sum", fdata[:, :n])
        assert all(bits_equal(rt.download(fdst, pe, (n,), np.float32), want) for pe in range(npes))
        rt.alltoall("float", fdst, fsrc, n)
        assert np.array_equal(rt.download_all(fdst, (npes * n * 4,), np.uint8), O.alltoall(fdata.view(np.uint8)))
        for p in (src, dst, fsrc, fdst):
            rt.free(p)


@pytest.mark.parametrize("npes", [5, 8, 16])
def test_large_source_fcollect_and_broadcast_across_several_chunks(npes, monkeypatch):
    """The large-source form of fcollect / broadcast walks the message in chunks of a few MiB, once per
    group of destinations: a message of several chunks plus a ragged rest, misaligned at both ends, must
    arrive whole on every member, with the bytes around the destination untouched."""
    monkeypatch.setenv("NVSHMEM_AMD_CACHEABLE_SOURCE_BYTES", "0")
    monkeypatch.setenv("NVSHMEM_AMD_CHUNKED_COPY_BYTES", "0")
    rng = np.random.default_rng(4100 + npes)
    nbytes = (9 << 20) + 1234
    with runtime(npes, (npes + 1) * (10 << 20) + (8 << 20)) as rt:
        src = rt.malloc(nbytes + 64); dst = rt.malloc(npes * nbytes + 256)
        data = rng.integers(0, 256, (npes, nbytes), dtype=np.uint8)
        for soff, doff in ((0, 0), (3, 21)):
            rt.upload_all(src, data, soff)
            rt.fill(dst, 0xCD, npes * nbytes + 256)
            note("chunked fcollect npes=%d bytes=%d soff=%d doff=%d" % (npes, nbytes, soff, doff))
            rt.fcollectmem(dst + doff, src + soff, nbytes)
            want = O.fcollect(data)
            for pe in (0, npes // 2, npes - 1):
                got = rt.download(dst, pe, (npes * nbytes + doff + 32,), np.uint8)
                assert np.array_equal(got[doff:doff + npes * nbytes], want[pe]), (pe, soff, doff)
                assert (got[:doff] == 0xCD).all() and (got[doff + npes * nbytes:] == 0xCD).all()
            root = npes - 2
            rt.fill(dst, 0xCD, npes * nbytes + 256)
            note("chunked broadcast npes=%d bytes=%d root=%d" % (npes, nbytes, root))
            rt.broadcastmem(dst + doff, src + soff, nbytes, root)
            got = rt.download_all(dst, (nbytes + doff + 32,), np.uint8)
            assert np.array_equal(got[:, doff:doff + nbytes], O.broadcast(data, root)), (soff, doff)
            assert (got[:, :doff] == 0xCD).all() and (got[:, doff + nbytes:] == 0xCD).all()
        rt.free(src); rt.free(dst)


@pytest.mark.parametrize("npes", [3, 5, 12, 24, 32, 33, 48, 64])
def test_lds_staged_allreduce_for_every_team_size_class(npes, monkeypatch):
    """The LDS-staged allreduce serves teams of 3 to 64 members once the sources outgrow the cache
    (NVSHMEM_AMD_LDS_REDUCE_BYTES, read at init): two members per wavefront up to 32, four beyond, 32 as a
    compile-time size.  With the threshold at zero small messages take it too: ragged counts, buffers that
    do not start on a 1 KiB boundary, in place, order-sensitive fp32 and bf16 sums, NaN-carrying max."""
    monkeypatch.setenv("NVSHMEM_AMD_LDS_REDUCE_BYTES", "0")
    monkeypatch.setenv("NVSHMEM_AMD_TWO_STEP_REDUCE_MEMBERS", "0")     # (the two-step form has its own test)
    _allreduce_battery(npes, np.random.default_rng(7000 + npes), "lds")


@pytest.mark.parametrize("npes", [4, 16, 24, 33, 64])
def test_two_step_allreduce(npes, monkeypatch):
    """Large teams with sources beyond the cache fold into member 0's destination and broadcast that
    (NVSHMEM_AMD_TWO_STEP_REDUCE_MEMBERS / _BYTES, read at init).  With the thresholds lowered every size and
    team takes that path: the same battery as the fused kernel - ragged counts, misaligned buffers, in place,
    NaN-carrying max, bf16, int64, families of ragged teams - must come out bit for bit the same."""
    monkeypatch.setenv("NVSHMEM_AMD_LDS_REDUCE_BYTES", "0")
    monkeypatch.setenv("NVSHMEM_AMD_CACHEABLE_SOURCE_BYTES", "0")
    monkeypatch.setenv("NVSHMEM_AMD_CHUNKED_COPY_BYTES", "0")
    monkeypatch.setenv("NVSHMEM_AMD_TWO_STEP_REDUCE_MEMBERS", "2")
    monkeypatch.setenv("NVSHMEM_AMD_TWO_STEP_REDUCE_BYTES", "0")
    _allreduce_battery(npes, np.random.default_rng(7100 + npes), "two-step")


def _allreduce_battery(npes, rng, tag):
    with runtime(npes, 16 << 20) as rt:
        cap = 40000
        src = rt.malloc(cap * 8 + 1024); dst = rt.malloc(cap * 8 + 1024)
        for n, off in ((1, 0), (255, 16), (256, 0), (4099, 48), (cap, 0), (30001, 1008)):
            f = (rng.standard_normal((npes, n)) * 10.0 ** rng.integers(-3, 4, (npes, n))).astype(np.float32)
            rt.upload_all(src, f, off)
            rt.fill(dst, 0xCD, cap * 8 + 1024)
            note("%s allreduce npes=%d float sum n=%d off=%d" % (tag, npes, n, off))
            rt.reduce("float", "sum", dst + off, src + off, n)
            want = O.reduce("f32", "sum", f)
            got = rt.download_all(dst, ((off + n * 4 + 64) // 4,), np.uint32)
            for pe in range(npes):
                assert bits_equal(got[pe, off // 4:off // 4 + n], want.view(np.uint32)), (n, off, pe)
            assert (got[:, :off // 4] == 0xCDCDCDCD).all() and (got[:, off // 4 + n:] == 0xCDCDCDCD).all()
        n = 12345
        f = rng.standard_normal((npes, n)).astype(np.float32)
        f[rng.integers(0, npes, 50), rng.integers(0, n, 50)] = np.nan
        f[rng.integers(0, npes, 50), rng.integers(0, n, 50)] = -0.0
        rt.upload_all(src, f)
        note("%s allreduce npes=%d float max with NaN, in place" % (tag, npes))
        rt.reduce("float", "max", src, src, n)
        want = O.reduce("f32", "max", f)
        assert all(bits_equal(rt.download(src, pe, (n,), np.float32), want) for pe in (0, npes // 2, npes - 1))
        b = (rng.standard_normal((npes, n)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        rt.upload_all(src, b)
        rt.reduce("bfloat16", "sum", dst, src, n)
        assert bits_equal(rt.download(dst, npes - 1, (n,), np.uint16), O.reduce("bf16", "sum", b))
        x = rng.integers(-2**63, 2**63 - 1, (npes, n), dtype=np.int64)
        rt.upload_all(src, x)
        rt.reduce("int64", "xor", dst, src, n)
        assert np.array_equal(rt.download(dst, 1, (n,), np.int64), O.reduce("i64", "xor", x))
        # a family of ragged teams on one handle: rows of a 2-D split, the last one shorter
        xr = 5 if npes > 5 else 2
        xt, yt = rt.team_split_2d(N.TEAM_WORLD, xr)
        f = (rng.standard_normal((npes, n)) * 10.0 ** rng.integers(-3, 4, (npes, n))).astype(np.float32)
        rt.upload_all(src, f)
        note("%s allreduce npes=%d rows of %d" % (tag, npes, xr))
        rt.reduce("float", "sum", dst, src, n, team=xt)
        for r0 in range(0, npes, xr):
            members = list(range(r0, min(r0 + xr, npes)))
            want = O.reduce("f32", "sum", f[members])
            for pe in (members[0], members[-1]):
                assert bits_equal(rt.download(dst, pe, (n,), np.float32), want), (r0, pe)
        rt.reduce("float", "sum", dst, src, n, team=yt)       # columns: strided members
        for c in (0, xr - 1):
            members = list(range(c, npes, xr))
            want = O.reduce("f32", "sum", f[members])
            assert bits_equal(rt.download(dst, members[-1], (n,), np.float32), want), c
        rt.team_destroy(xt); rt.team_destroy(yt)
        rt.free(src); rt.free(dst)
