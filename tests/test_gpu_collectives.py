"""GPU parity of reduce / fcollect / alltoall (a8-a11) through the C ABI against the CPU oracle.
Integer results, copies and permutations must be bit-exact.  Floating-point reductions use the
fixed PE order 0..n-1 in the element type, so they are compared bit for bit as well, which is
inside the stated tolerances (fp32: 1 ulp, bf16: 1e-2 relative); the tolerance check is kept
explicit for the configurations the metric is quoted on."""
import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import bits_equal, note, runtime
from nvshmem_amd.host import RMA_TYPES, REDUCE_TYPES_BITWISE, REDUCE_TYPES_STANDARD

pytestmark = pytest.mark.gpu


def _random_storage(kind, shape, rng, op):
    dt = O.NP_STORAGE[kind]
    if kind in ("f32", "f64"):
        x = rng.standard_normal(shape).astype(dt)
        if op == "prod":
            x = (1.0 + 0.25 * x).astype(dt)
        return x
    if kind in ("bf16", "f16"):
        f = rng.standard_normal(shape).astype(np.float32)
        if op == "prod":
            f = (1.0 + 0.25 * f).astype(np.float32)
        if kind == "f16":
            return f.astype(np.float16).view(np.uint16)
        u = f.view(np.uint32)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    info = np.iinfo(dt)
    return rng.integers(info.min, info.max, size=shape, dtype=dt, endpoint=True)


@pytest.fixture(scope="module", params=["gather", "lds"])
def rt8(request):
    """Every test of this module runs with both allreduce kernels: the default choice (the gather
    kernel at these sizes) and the LDS-staged kernel forced by NVSHMEM_AMD_LDS_REDUCE_BYTES=0."""
    import os
    old = os.environ.get("NVSHMEM_AMD_LDS_REDUCE_BYTES")
    if request.param == "lds":
        os.environ["NVSHMEM_AMD_LDS_REDUCE_BYTES"] = "0"
    try:
        with runtime(8, 1 << 28) as r:
            yield r
    finally:
        if old is None:
            os.environ.pop("NVSHMEM_AMD_LDS_REDUCE_BYTES", None)
        else:
            os.environ["NVSHMEM_AMD_LDS_REDUCE_BYTES"] = old


# ---------------------------------------------------------------------------------------------
# config 1 exactly: int32 sum, 8 PEs, 1M elements per PE, values in [-2^20, 2^20], seed 1
# ---------------------------------------------------------------------------------------------
def test_config1_int32_sum_reduce_bit_exact(rt8):
    n = 1 << 20
    src = rt8.malloc(n * 4); dst = rt8.malloc(n * 4)
    data = O.fill_all("i32", 8, n, 1)
    rt8.upload_all(src, data)
    note("config 1: nvshmem_int32_sum_reduce n=%d" % n)
    rt8.reduce("int32", "sum", dst, src, n)
    want = O.reduce("i32", "sum", data)
    got = rt8.download_all(dst, (n,), np.int32)
    for pe in range(8):
        assert np.array_equal(got[pe], want), pe
    # reference known answer (examples/ring-reduce.cu:242-248): src[i] = i everywhere -> i * npes
    rt8.upload_all(src, np.tile(np.arange(n, dtype=np.int32), (8, 1)))
    rt8.reduce("int", "sum", dst, src, n)
    assert np.array_equal(rt8.download(dst, 5, (n,), np.int32), np.arange(n, dtype=np.int32) * 8)
    rt8.free(src); rt8.free(dst)


# ---------------------------------------------------------------------------------------------
# every typed entry point of the reduce matrix (25 names x their operators)
# ---------------------------------------------------------------------------------------------
def _reduce_cases():
    for op in ("and", "or", "xor"):
        for t in REDUCE_TYPES_BITWISE:
            yield t, op
    for op in ("max", "min", "sum", "prod"):
        for t in REDUCE_TYPES_STANDARD:
            yield t, op


def test_every_typed_reduce_entry_point(rt8):
    n = 1531                      # odd: exercises the tail behind the last 16-byte vector
    rng = np.random.default_rng(42)
    src = rt8.malloc(n * 8); dst = rt8.malloc(n * 8)
    count = 0
    for t, op in _reduce_cases():
        np_dt, kind = RMA_TYPES[t]
        data = _random_storage(kind, (8, n), rng, op)
        rt8.upload_all(src, data)
        note("nvshmem_%s_%s_reduce n=%d" % (t, op, n))
        rt8.reduce(t, op, dst, src, n)
        want = O.reduce(kind, op, data)
        got = rt8.download_all(dst, (n,), data.dtype)
        for pe in range(8):
            assert bits_equal(got[pe], want), (t, op, pe)
        count += 1
    assert count == 3 * 14 + 4 * 24
    rt8.free(src); rt8.free(dst)


@pytest.mark.parametrize("t,kind,op", [("float", "f32", "max"), ("float", "f32", "min"),
                                       ("bfloat16", "bf16", "max"), ("double", "f64", "min")])
def test_min_max_with_nan_and_signed_zero_follow_the_operand_rule(rt8, t, kind, op):
    n = 4096
    rng = np.random.default_rng(9)
    f = rng.standard_normal((8, n)).astype(np.float32)
    f[rng.random((8, n)) < 0.1] = np.nan
    f[rng.random((8, n)) < 0.1] = 0.0
    f[rng.random((8, n)) < 0.1] = -0.0
    if kind == "f32":
        data = f
    elif kind == "f64":
        data = f.astype(np.float64)
    else:
        data = (f.view(np.uint32) >> 16).astype(np.uint16)   # truncation keeps NaN / zeros
    src = rt8.malloc(n * 8); dst = rt8.malloc(n * 8)
    rt8.upload_all(src, data)
    note("nan/zero %s %s" % (t, op))
    rt8.reduce(t, op, dst, src, n)
    want = O.reduce(kind, op, data)
    assert bits_equal(rt8.download(dst, 3, (n,), data.dtype), want)
    rt8.free(src); rt8.free(dst)


def test_reduce_in_place_unaligned_stream_and_sizes(rt8):
    from nvshmem_amd import hip
    rng = np.random.default_rng(1)
    buf = rt8.malloc(1 << 22)
    out = rt8.malloc(1 << 22)
    s = hip.Stream()
    for n in (1, 2, 3, 4, 5, 63, 64, 65, 1023, 4099, 262144 + 3):
        data = rng.standard_normal((8, n)).astype(np.float32)
        want = O.reduce("f32", "sum", data)
        # in place (dest == source), on a stream
        rt8.upload_all(buf, data)
        note("in-place float sum n=%d" % n)
        rt8.reduce("float", "sum", buf, buf, n, stream=s)
        s.synchronize()
        for pe in (0, 7):
            assert bits_equal(rt8.download(buf, pe, (n,), np.float32), want), (n, pe)
        # buffers offset by one element: the element-at-a-time kernel
        rt8.upload_all(buf, data, 4)
        note("unaligned float sum n=%d" % n)
        rt8.reduce("float", "sum", out + 4, buf + 4, n)
        assert bits_equal(rt8.download(out, 6, (n,), np.float32, 4), want), n
    # n == 0 is a no-op that succeeds
    rt8.reduce("float", "sum", out, buf, 0)
    s.destroy()
    rt8.free(buf); rt8.free(out)


def test_collective_argument_errors_are_reported(rt8):
    a = rt8.malloc(4096); b = rt8.malloc(4096)
    with pytest.raises(N.host.NvshmemError, match="team"):
        rt8.reduce("float", "sum", a, b, 16, team=20)
    with pytest.raises(N.host.NvshmemError, match="not a symmetric address"):
        rt8.reduce("float", "sum", 0x4000, b, 16)
    with pytest.raises(N.host.NvshmemError, match="overlap"):
        rt8.reduce("float", "sum", a + 16, a, 16)
    with pytest.raises(N.host.NvshmemError, match="heap slice"):
        rt8.reduce("float", "sum", a, b, 1 << 40)
    with pytest.raises(N.host.NvshmemError, match="overlap"):
        rt8.alltoallmem(a, a + 8, 64)
    with pytest.raises(N.host.NvshmemError):
        rt8.fcollectmem(a, b, 1 << 40)
    rt8.free(a); rt8.free(b)


# ---------------------------------------------------------------------------------------------
# fcollect / alltoall: ragged byte counts, misaligned buffers, typed names
# ---------------------------------------------------------------------------------------------
def test_fcollect_alltoall_ragged_and_misaligned(rt8):
    rng = np.random.default_rng(2)
    cap = 1 << 21
    src = rt8.malloc(cap + 64); dst = rt8.malloc(8 * cap + 64)
    for seg in (1, 5, 16, 17, 255, 4096, 4097, 32768 + 9, 200000):
        for soff, doff in ((0, 0), (1, 0), (0, 3), (7, 9)):
            data = rng.integers(0, 256, (8, seg), dtype=np.uint8)
            rt8.fill(dst, 0xCD, 8 * cap + 64)
            rt8.upload_all(src, data, soff)
            note("fcollectmem seg=%d soff=%d doff=%d" % (seg, soff, doff))
            rt8.fcollectmem(dst + doff, src + soff, seg)
            got = rt8.download_all(dst, (8 * seg + 32,), np.uint8)
            assert np.array_equal(got[:, doff:doff + 8 * seg], O.fcollect(data)), (seg, soff, doff)
            assert (got[:, :doff] == 0xCD).all() and (got[:, doff + 8 * seg:] == 0xCD).all()
            data = rng.integers(0, 256, (8, 8 * seg), dtype=np.uint8)
            if 8 * seg + soff <= cap:
                rt8.fill(dst, 0xCD, 8 * cap + 64)
                rt8.upload_all(src, data, soff)
                note("alltoallmem seg=%d soff=%d doff=%d" % (seg, soff, doff))
                rt8.alltoallmem(dst + doff, src + soff, seg)
                got = rt8.download_all(dst, (8 * seg + 32,), np.uint8)
                assert np.array_equal(got[:, doff:doff + 8 * seg], O.alltoall(data)), (seg, soff, doff)
                assert (got[:, :doff] == 0xCD).all() and (got[:, doff + 8 * seg:] == 0xCD).all()
    rt8.free(src); rt8.free(dst)


def test_typed_fcollect_alltoall_names(rt8):
    rng = np.random.default_rng(3)
    n = 333
    src = rt8.malloc(8 * n * 8); dst = rt8.malloc(8 * n * 8)
    for t, (np_dt, kind) in RMA_TYPES.items():
        es = np.dtype(np_dt).itemsize
        data = rng.integers(0, 256, (8, 8 * n * es), dtype=np.uint8)
        rt8.upload_all(src, data)
        note("nvshmem_%s_alltoall / fcollect" % t)
        rt8.alltoall(t, dst, src, n)
        assert np.array_equal(rt8.download_all(dst, (8 * n * es,), np.uint8), O.alltoall(data)), t
        rt8.fcollect(t, dst, src, n)
        assert np.array_equal(rt8.download_all(dst, (8 * n * es,), np.uint8),
                              O.fcollect(data[:, :n * es])), t
    rt8.free(src); rt8.free(dst)


# ---------------------------------------------------------------------------------------------
# in-kernel collectives (one thread group per PE) in the three scopes
# ---------------------------------------------------------------------------------------------
DEVICE_PAIRS = [("i32", "sum"), ("i64", "xor"), ("f32", "sum"), ("f32", "max"), ("bf16", "sum"),
                ("bf16", "max"), ("u64", "and"), ("f64", "prod"), ("i16", "min")]


@pytest.mark.parametrize("scope,threads", [(N.SCOPE_THREAD, 64), (N.SCOPE_WARP, 128), (N.SCOPE_BLOCK, 512)])
def test_device_scope_collectives(rt8, scope, threads):
    perf = rt8.perftest()
    rng = np.random.default_rng(scope)
    n = 3001
    src = rt8.malloc(8 * n * 8); dst = rt8.malloc(8 * n * 8)
    for kind, op in DEVICE_PAIRS:
        data = _random_storage(kind, (8, n), rng, op)
        rt8.upload_all(src, data)
        note("device reduce %s %s scope=%d" % (kind, op, scope))
        assert perf.nvshmem_perftest_device_reduce(N.DTYPES[kind], N.OPS[op], dst, src, n, scope,
                                                   threads, None) == 0
        rt8.sync()
        want = O.reduce(kind, op, data)
        got = rt8.download_all(dst, (n,), data.dtype)
        for pe in range(8):
            assert bits_equal(got[pe], want), (kind, op, pe)
    # in place
    data = _random_storage("f32", (8, n), rng, "sum")
    rt8.upload_all(src, data)
    assert perf.nvshmem_perftest_device_reduce(N.DTYPES["f32"], N.OPS["sum"], src, src, n, scope,
                                               threads, None) == 0
    rt8.sync()
    assert bits_equal(rt8.download(src, 4, (n,), np.float32), O.reduce("f32", "sum", data))
    # buffers offset by one element: the element-at-a-time path of the in-kernel reduce
    rt8.upload_all(src, data, 4)
    assert perf.nvshmem_perftest_device_reduce(N.DTYPES["f32"], N.OPS["sum"], dst + 4, src + 4, n, scope,
                                               threads, None) == 0
    rt8.sync()
    assert bits_equal(rt8.download(dst, 6, (n,), np.float32, 4), O.reduce("f32", "sum", data))
    assert perf.nvshmem_perftest_device_reduce(N.DTYPES["f32"], N.OPS["xor"], dst, src, n, scope,
                                               threads, None) == 3   # NVSHMEMX_ERROR_NOT_SUPPORTED
    for seg in (1, 100, 4097):
        data = rng.integers(0, 256, (8, 8 * seg), dtype=np.uint8)
        rt8.upload_all(src, data)
        note("device alltoall/fcollect seg=%d scope=%d" % (seg, scope))
        assert perf.nvshmem_perftest_device_alltoall(dst, src, seg, scope, threads, None) == 0
        rt8.sync()
        assert np.array_equal(rt8.download_all(dst, (8 * seg,), np.uint8), O.alltoall(data))
        assert perf.nvshmem_perftest_device_fcollect(dst, src, seg, scope, threads, None) == 0
        rt8.sync()
        assert np.array_equal(rt8.download_all(dst, (8 * seg,), np.uint8), O.fcollect(data[:, :seg]))
    rt8.free(src); rt8.free(dst)
