"""GPU parity of broadcast and reducescatter through the C ABI against the CPU oracle: bit-exact for
bytes and integers; floating-point reducescatter folds in the fixed order acc = op(acc, x_p), p =
0..n-1, in the element type, so it is compared bit for bit as well (inside fp32 1 ulp, bf16 1e-2)."""
import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import bits_equal, note, runtime
from nvshmem_amd.host import RMA_TYPES, REDUCE_TYPES_BITWISE, REDUCE_TYPES_STANDARD
from test_gpu_collectives import _random_storage, _reduce_cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt8():
    with runtime(8, 1 << 28) as r:
        yield r


# ---------------------------------------------------------------------------------------------
# broadcast
# ---------------------------------------------------------------------------------------------
def test_broadcast_reference_known_answer(rt8):
    # examples/ring-bcast.cu:44-72: PE 0 holds data[i] = mype + i = i, every PE ends with data[i] = i
    n = 1 << 20
    buf = rt8.malloc(n * 4); dst = rt8.malloc(n * 4)
    data = np.stack([(pe + np.arange(n)).astype(np.int32) for pe in range(8)])
    rt8.upload_all(buf, data)
    note("nvshmem_int_broadcast n=%d root=0" % n)
    rt8.broadcast("int", dst, buf, n, 0)
    got = rt8.download_all(dst, (n,), np.int32)
    assert all(np.array_equal(got[pe], np.arange(n, dtype=np.int32)) for pe in range(8))
    rt8.free(buf); rt8.free(dst)


def test_broadcastmem_ragged_misaligned_every_root_and_in_place(rt8):
    rng = np.random.default_rng(12)
    cap = 1 << 20
    src = rt8.malloc(cap + 64); dst = rt8.malloc(cap + 64)
    root = 0
    for nbytes in (1, 5, 16, 17, 255, 1024, 4097, 32768 + 9, 300001):
        for soff, doff in ((0, 0), (1, 0), (0, 3), (7, 9)):
            root = (root + 3) % 8
            data = rng.integers(0, 256, (8, nbytes), dtype=np.uint8)
            rt8.fill(dst, 0xCD, cap + 64)
            rt8.upload_all(src, data, soff)
            note("broadcastmem bytes=%d soff=%d doff=%d root=%d" % (nbytes, soff, doff, root))
            rt8.broadcastmem(dst + doff, src + soff, nbytes, root)
            got = rt8.download_all(dst, (nbytes + 32,), np.uint8)
            assert np.array_equal(got[:, doff:doff + nbytes], O.broadcast(data, root)), (nbytes, soff, doff)
            assert (got[:, :doff] == 0xCD).all() and (got[:, doff + nbytes:] == 0xCD).all()
            # the sources are untouched
            assert np.array_equal(rt8.download_all(src, (nbytes,), np.uint8, soff), data)
    # in place: dest == source; the root keeps its data, everybody else receives it
    from nvshmem_amd import hip
    s = hip.Stream()
    data = rng.integers(0, 256, (8, 70001), dtype=np.uint8)
    rt8.upload_all(src, data, 5)
    note("broadcastmem in place on a stream root=6")
    rt8.broadcastmem(src + 5, src + 5, 70001, 6, stream=s)
    s.synchronize()
    assert np.array_equal(rt8.download_all(src, (70001,), np.uint8, 5), O.broadcast(data, 6))
    s.destroy()
    rt8.free(src); rt8.free(dst)


def test_typed_broadcast_names(rt8):
    rng = np.random.default_rng(13)
    n = 777
    src = rt8.malloc(n * 8); dst = rt8.malloc(n * 8)
    for k, (t, (np_dt, kind)) in enumerate(RMA_TYPES.items()):
        es = np.dtype(np_dt).itemsize
        data = rng.integers(0, 256, (8, n * es), dtype=np.uint8)
        rt8.upload_all(src, data)
        note("nvshmem_%s_broadcast root=%d" % (t, k % 8))
        rt8.broadcast(t, dst, src, n, k % 8)
        assert np.array_equal(rt8.download_all(dst, (n * es,), np.uint8), O.broadcast(data, k % 8)), t
    rt8.free(src); rt8.free(dst)


def test_broadcast_argument_errors(rt8):
    a = rt8.malloc(4096); b = rt8.malloc(4096)
    with pytest.raises(N.host.NvshmemError, match="root"):
        rt8.broadcastmem(a, b, 64, 8)
    with pytest.raises(N.host.NvshmemError, match="root"):
        rt8.broadcastmem(a, b, 64, -1)
    with pytest.raises(N.host.NvshmemError, match="overlap"):
        rt8.broadcastmem(a + 8, a, 64, 0)
    with pytest.raises(N.host.NvshmemError, match="team"):
        rt8.broadcast("float", a, b, 16, 0, team=20)
    with pytest.raises(N.host.NvshmemError):
        rt8.broadcastmem(a, b, 1 << 40, 0)
    rt8.broadcastmem(a, b, 0, 0)      # nothing to do
    rt8.free(a); rt8.free(b)


# ---------------------------------------------------------------------------------------------
# reducescatter
# ---------------------------------------------------------------------------------------------
def test_every_typed_reducescatter_entry_point(rt8):
    rng = np.random.default_rng(43)
    src = rt8.malloc(8 * 2048 * 8); dst = rt8.malloc(2048 * 8)
    count = 0
    for t, op in _reduce_cases():
        np_dt, kind = RMA_TYPES[t]
        # 1536 elements: blocks of whole 16-byte vectors for every element size (the LDS-staged
        # kernel); 1531 elements: the element-at-a-time kernel
        for n in (1536, 1531) if count % 3 == 0 else (1536,):
            data = _random_storage(kind, (8, 8 * n), rng, op)
            rt8.upload_all(src, data)
            note("nvshmem_%s_%s_reducescatter n=%d" % (t, op, n))
            rt8.reducescatter(t, op, dst, src, n)
            want = O.reducescatter(kind, op, data)
            got = rt8.download_all(dst, (n,), data.dtype)
            assert bits_equal(got, want), (t, op, n)
        count += 1
    assert count == 3 * 14 + 4 * 24
    rt8.free(src); rt8.free(dst)


def test_reducescatter_operand_order_with_nan(rt8):
    # max(a, b) = (a > b) ? a : b folded as acc = op(acc, x): a NaN met in the middle is dropped by
    # the next comparison, unlike in reduce, whose order is acc = op(x, acc)
    n = 4096
    rng = np.random.default_rng(10)
    f = rng.standard_normal((8, 8 * n)).astype(np.float32)
    f[rng.random((8, 8 * n)) < 0.15] = np.nan
    f[rng.random((8, 8 * n)) < 0.1] = 0.0
    f[rng.random((8, 8 * n)) < 0.1] = -0.0
    src = rt8.malloc(8 * n * 4); dst = rt8.malloc(n * 4)
    for op in ("max", "min"):
        rt8.upload_all(src, f)
        note("reducescatter float %s with NaN / signed zeros" % op)
        rt8.reducescatter("float", op, dst, src, n)
        want = O.reducescatter("f32", op, f)
        assert bits_equal(rt8.download_all(dst, (n,), np.float32), want)
        as_reduce = O.reduce("f32", op, f).reshape(8, n)
        assert not bits_equal(as_reduce, want), "input does not tell the two operand orders apart"
    rt8.free(src); rt8.free(dst)


def test_reducescatter_sizes_offsets_stream(rt8):
    from nvshmem_amd import hip
    rng = np.random.default_rng(5)
    src = rt8.malloc(1 << 24); dst = rt8.malloc(1 << 21)
    s = hip.Stream()
    for n in (1, 3, 4, 5, 64, 252, 256, 260, 4100, 65536 + 4, 262144):
        data = rng.standard_normal((8, 8 * n)).astype(np.float32)
        want = O.reducescatter("f32", "sum", data)
        for soff, doff in ((0, 0), (16, 48), (4, 0), (0, 4)):
            rt8.fill(dst, 0xCD, 1 << 21)
            rt8.upload_all(src, data, soff)
            note("reducescatter float sum n=%d soff=%d doff=%d" % (n, soff, doff))
            rt8.reducescatter("float", "sum", dst + doff, src + soff, n, stream=s)
            s.synchronize()
            got = rt8.download_all(dst, (n + 16,), np.float32)
            lo = doff // 4
            assert bits_equal(got[:, lo:lo + n], want), (n, soff, doff)
            guard = np.delete(got.view(np.uint32), np.s_[lo:lo + n], axis=1)
            assert (guard == 0xCDCDCDCD).all(), (n, soff, doff)
    rt8.reducescatter("float", "sum", dst, src, 0)
    with pytest.raises(N.host.NvshmemError, match="overlap"):
        rt8.reducescatter("float", "sum", src + 64, src, 64)
    with pytest.raises(N.host.NvshmemError, match="heap slice"):
        rt8.reducescatter("float", "sum", dst, src, 1 << 40)
    s.destroy()
    rt8.free(src); rt8.free(dst)


# ---------------------------------------------------------------------------------------------
# in-kernel forms (one thread group per PE) in the three scopes
# ---------------------------------------------------------------------------------------------
SCATTER_PAIRS = [("i32", "sum"), ("f32", "sum"), ("f32", "max"), ("bf16", "sum"), ("u64", "xor")]


@pytest.mark.parametrize("scope,threads", [(N.SCOPE_THREAD, 64), (N.SCOPE_WARP, 128), (N.SCOPE_BLOCK, 512)])
def test_device_scope_broadcast_and_reducescatter(rt8, scope, threads):
    perf = rt8.perftest()
    rng = np.random.default_rng(20 + scope)
    n = 1003
    src = rt8.malloc(8 * n * 8 + 64); dst = rt8.malloc(n * 8 + 64)
    for kind, op in SCATTER_PAIRS:
        es = O.NP_STORAGE[kind]().itemsize
        for off in (0, es):     # vector path / element path
            data = _random_storage(kind, (8, 8 * n), rng, op)
            if kind == "f32" and op == "max":
                data[rng.random(data.shape) < 0.1] = np.nan
            rt8.upload_all(src, data, off)
            note("device reducescatter %s %s scope=%d off=%d" % (kind, op, scope, off))
            assert perf.nvshmem_perftest_device_reducescatter(N.DTYPES[kind], N.OPS[op], dst + off,
                                                              src + off, n, scope, threads, None) == 0
            rt8.sync()
            want = O.reducescatter(kind, op, data)
            assert bits_equal(rt8.download_all(dst, (n,), data.dtype, off), want), (kind, op, off)
    assert perf.nvshmem_perftest_device_reducescatter(N.DTYPES["f64"], N.OPS["sum"], dst, src, n, scope,
                                                      threads, None) == 3   # NVSHMEMX_ERROR_NOT_SUPPORTED
    for nbytes, root, off in ((1, 0, 0), (100, 3, 1), (4097, 7, 0), (8 * n, 5, 3)):
        data = rng.integers(0, 256, (8, nbytes), dtype=np.uint8)
        rt8.fill(dst, 0xCD, n * 8 + 64)
        rt8.upload_all(src, data, off)
        note("device broadcast bytes=%d root=%d scope=%d" % (nbytes, root, scope))
        assert perf.nvshmem_perftest_device_broadcast(dst, src + off, nbytes, root, scope, threads, None) == 0
        rt8.sync()
        got = rt8.download_all(dst, (nbytes + 16,), np.uint8)
        assert np.array_equal(got[:, :nbytes], O.broadcast(data, root))
        assert (got[:, nbytes:] == 0xCD).all()
    # in place: the root's own copy is skipped
    data = rng.integers(0, 256, (8, 5000), dtype=np.uint8)
    rt8.upload_all(src, data)
    assert perf.nvshmem_perftest_device_broadcast(src, src, 5000, 2, scope, threads, None) == 0
    rt8.sync()
    assert np.array_equal(rt8.download_all(src, (5000,), np.uint8), O.broadcast(data, 2))
    assert perf.nvshmem_perftest_device_broadcast(dst, src, 16, 8, scope, threads, None) != 0
    rt8.free(src); rt8.free(dst)
