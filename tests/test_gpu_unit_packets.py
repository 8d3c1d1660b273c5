"""The 64-byte line packets (f4: the reference's LL128 re-derived; compiled in only where a translation unit
defines NVSHMEMI_AMD_UNIT_PACKETS, as libnvshmem_amd_perftest_units.so is): in-kernel allreduce and
reducescatter of 257 B ... 3.5 KiB per member then travel as units of 56 payload bytes + flag word.  Bit-exact against the oracle over element types,
sizes around both ends of the range, odd offsets, in place, wavefront and block scope, and 40 rounds of
reduce / broadcast / fcollect / alltoall / reducescatter with data that changes every round (a torn or
stale unit would show)."""
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


def _units():
    from nvshmem_amd import _lib
    lib = _lib.load_perftest_units()
    assert lib.nvshmem_perftest_unit_packets_compiled() == 1
    assert _lib.load_perftest().nvshmem_perftest_unit_packets_compiled() == 0     # the default build has none
    return lib


def _data(rng, kind, shape):
    if kind in ("f32", "f64"):
        d = (1.0 + 0.25 * rng.standard_normal(shape)).astype(O.NP_STORAGE[kind])
        d[rng.random(shape) < 0.05] = np.nan
        return d
    if kind == "bf16":
        return (rng.standard_normal(shape).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    info = np.iinfo(O.NP_STORAGE[kind])
    return rng.integers(info.min, info.max, shape, dtype=O.NP_STORAGE[kind], endpoint=True)


@pytest.mark.parametrize("scope,threads", [(N.SCOPE_BLOCK, 256), (N.SCOPE_BLOCK, 1024), (N.SCOPE_WARP, 64)])
def test_reduce_and_reducescatter_through_line_packets(rt8, scope, threads):
    perf = _units()
    rng = np.random.default_rng(threads)
    src = rt8.malloc(1 << 17); dst = rt8.malloc(1 << 17)
    lanes = threads if scope == N.SCOPE_BLOCK else 64
    top = min(lanes // 4, 64) * 56                     # largest message the units carry for this group
    for kind, op, es in (("f32", "sum", 4), ("f32", "max", 4), ("bf16", "sum", 2), ("i64", "xor", 8), ("f64", "prod", 8),
                         ("i16", "min", 2)):
        for nbytes in sorted(set([264, 512, 56 * 9, 56 * 9 + es, 1024, 2048, top - es, top, top + es])):
            n = nbytes // es
            data = _data(rng, kind, (8, n))
            for off in (0, es):
                rt8.upload_all(src, data, off)
                note("unit reduce %s %s n=%d off=%d scope=%d threads=%d" % (kind, op, n, off, scope, threads))
                assert perf.nvshmem_perftest_device_reduce(N.DTYPES[kind], N.OPS[op], dst + off, src + off, n,
                                                           scope, threads, None) == 0
                rt8.sync()
                want = O.reduce(kind, op, data)
                got = rt8.download_all(dst, (n,), data.dtype, off)
                assert all(bits_equal(got[pe], want) for pe in range(8)), (kind, op, n, off)
            rt8.upload_all(src, data)                  # in place
            assert perf.nvshmem_perftest_device_reduce(N.DTYPES[kind], N.OPS[op], src, src, n, scope, threads, None) == 0
            rt8.sync()
            assert bits_equal(rt8.download(src, 5, (n,), data.dtype), O.reduce(kind, op, data))
    for kind, op, es in (("i32", "sum", 4), ("f32", "max", 4), ("bf16", "sum", 2), ("u64", "xor", 8)):
        for nbytes in (272, 1024, min(top, 2048)):
            n = nbytes // es
            data = _data(rng, "f32" if kind == "f32" else kind, (8, 8 * n))
            rt8.upload_all(src, data)
            note("unit reducescatter %s %s n=%d scope=%d" % (kind, op, n, scope))
            assert perf.nvshmem_perftest_device_reducescatter(N.DTYPES[kind], N.OPS[op], dst, src, n, scope, threads,
                                                              None) == 0
            rt8.sync()
            assert bits_equal(rt8.download_all(dst, (n,), data.dtype), O.reducescatter(kind, op, data)), (kind, n)
    assert all(rt8.read_timeout(pe)[0] == 0 for pe in range(8))
    rt8.free(src); rt8.free(dst)


def test_forty_rounds_of_changing_data_through_line_packets(rt8):
    from test_gpu_small_collectives import _expected_checks
    perf = _units()
    for n, fc_bytes in ((300, 64), (512, 256), (896, 8)):       # 1200, 2048 and 3584 bytes per member
        src = rt8.malloc(5000 * 4); dst = rt8.malloc(8 * 2052 + 5000 * 4); check = rt8.calloc(1, 8)
        note("coll sequence through line packets n=%d" % n)
        assert perf.nvshmem_perftest_coll_sequence(src, dst, check, n, fc_bytes, 40, 1, N.SCOPE_BLOCK, 256, None) == 0
        rt8.sync()
        got = rt8.download_all(check, (1,), np.uint64)[:, 0]
        assert np.array_equal(got, _expected_checks(8, n, fc_bytes, 40))
        assert all(rt8.read_timeout(pe)[0] == 0 for pe in range(8))
        for p in (src, dst, check):
            rt8.free(p)
