"""GPU parity of the small-message (packet) paths of the in-kernel collectives: sizes around the
switch-over points in every scope, and long unsynchronised sequences of reduce / broadcast /
fcollect with rotating roots, whose checksums only come out right if no PE ever overwrites a packet
buffer that another PE is still reading."""
import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import bits_equal, note, runtime

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt8():
    with runtime(8, 1 << 24) as r:
        yield r


def _gen(npes, r, n):
    me = np.arange(npes, dtype=np.uint64)[:, None]
    i = np.arange(n, dtype=np.uint64)[None, :]
    return ((me * np.uint64(1000003) + np.uint64(r * 7919) + i * np.uint64(31)) & np.uint64(0xFFFFFFFF)
            & np.uint64(0x7FFFFFFF)).astype(np.int32)


def _checksum(h, words):
    w = words.astype(np.uint32).astype(np.uint64)
    weights = np.arange(len(w), dtype=np.uint64) * np.uint64(2) + np.uint64(1)
    with np.errstate(over="ignore"):
        return (h * np.uint64(1000003) + (w * weights).sum(dtype=np.uint64)).astype(np.uint64)


def _expected_checks(npes, n, fc_bytes, rounds):
    h = np.zeros(npes, np.uint64)
    for r in range(rounds):
        data = _gen(npes, r, n)
        red = O.reduce("i32", "sum", data)
        bc = data[r % npes]
        fc = O.fcollect(data.view(np.uint8)[:, :fc_bytes])
        w = n // npes
        if w:
            block = np.ascontiguousarray(data[:, :w * npes])
            a2a = O.alltoall(block.view(np.uint8)).view(np.int32)
            rs = O.reducescatter("i32", "sum", block)
        for pe in range(npes):
            h[pe] = _checksum(h[pe], red)
            h[pe] = _checksum(h[pe], bc)
            h[pe] = _checksum(h[pe], fc[pe].view(np.int32))
            if w:
                h[pe] = _checksum(h[pe], a2a[pe])
                h[pe] = _checksum(h[pe], rs[pe])
    return h


def _uses_packets(what, nbytes, npes, scope, threads):
    """The library's rule for taking the packet path: one packet per lane of the thread group (a
    single thread takes up to 8), nvshmemi_amd_ll_fits / nvshmemi_amd_ll_reduce_group."""
    nthr = {N.SCOPE_BLOCK: threads, N.SCOPE_WARP: 64, N.SCOPE_THREAD: 1}[scope]
    lanes = max(nthr, 8)
    npk = (nbytes + 7) // 8
    if what == "broadcast":
        # (a wavefront or block whose (member, chunk) pairs need more than one round over its lanes pushes
        # with the fan-out copy instead when source and dest share their offset within 16 bytes, as the
        # buffers of these tests do)
        return nbytes <= 16384 and npk * (npes - 1 if scope == N.SCOPE_THREAD else 1) <= lanes and \
            (npk * (npes - 1) <= lanes or scope == N.SCOPE_THREAD)
    ok = nbytes <= 2048 and npk * 8 * npes <= 16384 and npk * (npes - 1) <= lanes
    if what in ("reduce", "reducescatter") and scope != N.SCOPE_THREAD:
        group = 1
        while group < npes:
            group *= 2
        ok = ok and group * npk <= nthr
    return ok


@pytest.mark.parametrize("scope,threads", [(N.SCOPE_BLOCK, 256), (N.SCOPE_WARP, 64), (N.SCOPE_THREAD, 64),
                                           (N.SCOPE_BLOCK, 1024)])
@pytest.mark.parametrize("n,fc_bytes,sync_between", [(2, 8, 0), (16, 64, 0), (64, 256, 0), (125, 500, 0),
                                                     (512, 2048, 0), (512, 4, 0), (4096, 2048, 0),
                                                     (5000, 2052, 1)])
def test_unsynchronised_sequences(rt8, scope, threads, n, fc_bytes, sync_between):
    # reduce uses packets up to 2048 bytes, broadcast up to 16384, fcollect up to 2048 per PE:
    # (4096, 2048) mixes a barrier-based reduce with packet broadcasts and fcollects; the last
    # case leaves the packet paths altogether and needs the barriers a program would need too
    perf = rt8.perftest()
    # a broadcast or fcollect that does not travel as packets writes into the other PEs' dst at
    # once, so - as in any NVSHMEM program - the PEs must have finished with dst before it starts
    if not (_uses_packets("broadcast", n * 4, 8, scope, threads) and
            _uses_packets("fcollect", fc_bytes, 8, scope, threads) and
            (n < 8 or _uses_packets("alltoall", (n // 8) * 4, 8, scope, threads))):
        sync_between = 1
    rounds = 6 if scope == N.SCOPE_THREAD and n > 1000 else 40
    src = rt8.malloc(5000 * 4); dst = rt8.malloc(8 * 2052 + 5000 * 4); check = rt8.calloc(1, 8)
    note("coll sequence n=%d fc=%d rounds=%d scope=%d threads=%d sync=%d" % (n, fc_bytes, rounds, scope, threads, sync_between))
    assert perf.nvshmem_perftest_coll_sequence(src, dst, check, n, fc_bytes, rounds, sync_between, scope,
                                               threads, None) == 0
    rt8.sync()
    got = rt8.download_all(check, (1,), np.uint64)[:, 0]
    want = _expected_checks(8, n, fc_bytes, rounds)
    assert np.array_equal(got, want), (got, want)
    flag, rec = rt8.read_timeout(0)
    assert flag == 0, rec
    for p in (src, dst, check):
        rt8.free(p)


@pytest.mark.parametrize("scope,threads", [(N.SCOPE_BLOCK, 256), (N.SCOPE_WARP, 128), (N.SCOPE_THREAD, 64)])
def test_sizes_around_the_switch_over(rt8, scope, threads):
    perf = rt8.perftest()
    rng = np.random.default_rng(scope)
    src = rt8.malloc(1 << 16); dst = rt8.malloc(1 << 18)
    for kind, op, es in (("f32", "sum", 4), ("bf16", "max", 2), ("f64", "prod", 8), ("i16", "min", 2), ("i64", "xor", 8)):
        for nbytes in (es, 3 * es, 64, 248, 256, 256 + es, 1024, 2048, 2048 + es):
            n = nbytes // es
            if kind in ("f32", "f64"):
                data = (1.0 + 0.25 * rng.standard_normal((8, n))).astype(O.NP_STORAGE[kind])
            elif kind == "bf16":
                data = (rng.standard_normal((8, n)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
            else:
                info = np.iinfo(O.NP_STORAGE[kind])
                data = rng.integers(info.min, info.max, (8, n), dtype=O.NP_STORAGE[kind], endpoint=True)
            for off in (0, es):           # aligned / one element off an 8-byte boundary
                rt8.upload_all(src, data, off)
                note("device reduce %s %s n=%d off=%d scope=%d" % (kind, op, n, off, scope))
                assert perf.nvshmem_perftest_device_reduce(N.DTYPES[kind], N.OPS[op], dst + off, src + off, n,
                                                           scope, threads, None) == 0
                rt8.sync()
                want = O.reduce(kind, op, data)
                got = rt8.download_all(dst, (n,), data.dtype, off)
                for pe in range(8):
                    assert bits_equal(got[pe], want), (kind, op, n, off, pe)
            # in place
            rt8.upload_all(src, data)
            assert perf.nvshmem_perftest_device_reduce(N.DTYPES[kind], N.OPS[op], src, src, n, scope,
                                                       threads, None) == 0
            rt8.sync()
            assert bits_equal(rt8.download(src, 3, (n,), data.dtype), O.reduce(kind, op, data))
    for kind, op, es in (("i32", "sum", 4), ("f32", "max", 4), ("bf16", "sum", 2), ("u64", "xor", 8)):
        for nbytes in (es, 3 * es, 64, 256, 256 + es, 2048):
            n = nbytes // es
            if kind == "f32":
                data = rng.standard_normal((8, 8 * n)).astype(np.float32)
                data[rng.random(data.shape) < 0.1] = np.nan
            elif kind == "bf16":
                data = (rng.standard_normal((8, 8 * n)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
            else:
                info = np.iinfo(O.NP_STORAGE[kind])
                data = rng.integers(info.min, info.max, (8, 8 * n), dtype=O.NP_STORAGE[kind], endpoint=True)
            for off in (0, es):
                rt8.upload_all(src, data, off)
                note("device reducescatter %s %s n=%d off=%d scope=%d" % (kind, op, n, off, scope))
                assert perf.nvshmem_perftest_device_reducescatter(N.DTYPES[kind], N.OPS[op], dst + off, src + off,
                                                                  n, scope, threads, None) == 0
                rt8.sync()
                assert bits_equal(rt8.download_all(dst, (n,), data.dtype, off), O.reducescatter(kind, op, data)), \
                    (kind, op, n, off)
    # 72 | 73 and 288 | 289: one packet per lane of a wavefront / a 256-thread block; beyond, and up to
    # 16384 bytes, the fan-out copy (whole vectors from 16 bytes on, edge bytes around them)
    for nbytes in (1, 7, 8, 9, 63, 72, 73, 288, 289, 511, 512, 513, 1167, 1168, 1169, 2047, 2048, 2049, 16384, 16385):
        # (3, 5): no common offset within 16 bytes, a copy per member; (5, 21): a common one, the fan-out
        # copy with bytes in front of its first whole vector
        for soff, doff in ((0, 0), (3, 5), (5, 21)):
            data = rng.integers(0, 256, (8, nbytes), dtype=np.uint8)
            rt8.fill(dst, 0xCD, 1 << 18)
            rt8.upload_all(src, data, soff)
            note("device fcollect / broadcast bytes=%d soff=%d doff=%d scope=%d" % (nbytes, soff, doff, scope))
            assert perf.nvshmem_perftest_device_fcollect(dst + doff, src + soff, nbytes, scope, threads, None) == 0
            rt8.sync()
            got = rt8.download_all(dst, (8 * nbytes + 32,), np.uint8)
            assert np.array_equal(got[:, doff:doff + 8 * nbytes], O.fcollect(data))
            assert (got[:, :doff] == 0xCD).all() and (got[:, doff + 8 * nbytes:] == 0xCD).all()
            if 8 * nbytes + soff <= (1 << 16):
                data8 = rng.integers(0, 256, (8, 8 * nbytes), dtype=np.uint8)
                rt8.fill(dst, 0xCD, 1 << 18)
                rt8.upload_all(src, data8, soff)
                assert perf.nvshmem_perftest_device_alltoall(dst + doff, src + soff, nbytes, scope, threads, None) == 0
                rt8.sync()
                got = rt8.download_all(dst, (8 * nbytes + 32,), np.uint8)
                assert np.array_equal(got[:, doff:doff + 8 * nbytes], O.alltoall(data8))
                assert (got[:, :doff] == 0xCD).all() and (got[:, doff + 8 * nbytes:] == 0xCD).all()
                rt8.upload_all(src, data, soff)
            rt8.fill(dst, 0xCD, 1 << 18)
            assert perf.nvshmem_perftest_device_broadcast(dst + doff, src + soff, nbytes, 6, scope, threads, None) == 0
            rt8.sync()
            got = rt8.download_all(dst, (nbytes + 32,), np.uint8)
            assert np.array_equal(got[:, doff:doff + nbytes], O.broadcast(data, 6))
            assert (got[:, :doff] == 0xCD).all() and (got[:, doff + nbytes:] == 0xCD).all()
    rt8.free(src); rt8.free(dst)
