"""GPU parity at the full sizes of the headline configurations (3 and 4), compared directly with
the CPU oracle on the same seeded inputs, plus size-independent properties."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_util import bits_equal, note, runtime

pytestmark = pytest.mark.gpu


def _ulp_distance_f32(a, b):
    ia = a.view(np.int32).astype(np.int64); ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7FFFFFFF), ia); ib = np.where(ib < 0, -(ib & 0x7FFFFFFF), ib)
    return np.abs(ia - ib)


def test_config3_allreduce_64M_elements_per_pe():
    n = 1 << 26
    with runtime(8, (n * 8) * 2 + (1 << 20)) as rt:
        src = rt.malloc(n * 8); dst = rt.malloc(n * 8)
        # fp32 ~N(0,1), seed 3: sum and max
        data = O.fill_all("f32", 8, n, 3)
        rt.upload_all(src, data)
        for op in ("sum", "max"):
            note("config 3: float %s n=2^26" % op)
            rt.reduce("float", op, dst, src, n)
            want = O.reduce("f32", op, data)
            for pe in range(8):
                got = rt.download(dst, pe, (n,), np.float32)
                # stated tolerance: 1 ulp with the fixed PE order; the kernel is in fact bit-identical
                assert _ulp_distance_f32(got, want).max() <= 1
                assert bits_equal(got, want), (op, pe)
        # bf16 = RNE(fp32 N(0,1)), seed 4: sum and max
        data = O.fill_all("bf16", 8, n, 4)
        rt.upload_all(src, data)
        for op in ("sum", "max"):
            note("config 3: bfloat16 %s n=2^26" % op)
            rt.reduce("bfloat16", op, dst, src, n)
            want = O.reduce("bf16", op, data)
            wf = (want.astype(np.uint32) << 16).view(np.float32)
            for pe in (0, 3, 7):
                got = rt.download(dst, pe, (n,), np.uint16)
                gf = (got.astype(np.uint32) << 16).view(np.float32)
                # stated tolerance: 1e-2 relative (guarded near zero); the kernel is bit-identical
                assert (np.abs(gf - wf) <= 1e-2 * np.maximum(np.abs(wf), 1e-3)).all()
                assert bits_equal(got, want), (op, pe)
        # int64 uniform bits, seed 5: xor, in place as well
        data = O.fill_all("u64", 8, n, 5).view(np.int64)
        rt.upload_all(src, data)
        note("config 3: int64 xor n=2^26")
        rt.reduce("int64", "xor", dst, src, n)
        want = O.reduce("i64", "xor", data)
        for pe in range(8):
            assert np.array_equal(rt.download(dst, pe, (n,), np.int64), want), pe
        # property: xor-reducing the result with itself in place gives zero on an even team
        rt.reduce("int64", "xor", dst, dst, n)
        assert not rt.download(dst, 2, (n,), np.int64).any()
        rt.free(src); rt.free(dst)


@pytest.mark.parametrize("tname,es", [("float", 4), ("int64", 8)])
def test_config4_fcollect_alltoall_16_pes_4M_elements(tname, es):
    n = 1 << 22
    with runtime(16, n * es * 18 + (1 << 20)) as rt:
        src = rt.malloc(n * es); fdst = rt.malloc(16 * n * es); adst = rt.malloc(n * es)
        data = O.fill_all("u64", 16, n * es // 8, 6).view(np.uint8).reshape(16, -1)
        rt.upload_all(src, data)
        note("config 4: %s alltoall block=2^18" % tname)
        rt.alltoall(tname, adst, src, n // 16)
        got = rt.download_all(adst, (n * es,), np.uint8)
        assert np.array_equal(got, O.alltoall(data))
        # property: alltoall is an involution
        rt.alltoall(tname, src, adst, n // 16)
        assert np.array_equal(rt.download_all(src, (n * es,), np.uint8), data)
        note("config 4: %s fcollect n=2^22" % tname)
        rt.fcollect(tname, fdst, src, n)
        want = data.reshape(-1)
        for pe in range(16):
            assert np.array_equal(rt.download(fdst, pe, (16 * n * es,), np.uint8), want), pe
        rt.free(src); rt.free(fdst); rt.free(adst)


def test_host_put_and_get_beyond_the_cache_size():
    """Host-initiated transfers of more than 128 MiB between device buffers run on the library's own
    copy kernel instead of hipMemcpyAsync: every mutual alignment class once, host memory on the
    other side still works, bytes around the destination untouched."""
    import ctypes as C
    from nvshmem_amd import hip
    size = (128 << 20) + 4099
    rng = np.random.default_rng(9)
    with runtime(4, 2 * size + (64 << 20)) as rt:
        a = rt.malloc(size + 64); b = rt.malloc(size + 64)
        data = rng.integers(0, 256, size + 32, dtype=np.uint8)
        rt.upload(a, 0, data)
        s = hip.Stream()
        for soff, doff in ((0, 0), (3, 1), (16, 5)):
            rt.fill(b, 0xCD, size + 64)
            note("host put of %d bytes soff=%d doff=%d" % (size, soff, doff))
            rt.lib.nvshmemx_putmem_on_stream(b + doff, a + soff, size, 2, s.ptr)    # PE 0's a -> PE 2's b
            s.synchronize()
            got = rt.download(b, 2, (size + 48,), np.uint8)
            assert np.array_equal(got[doff:doff + size], data[soff:soff + size]), (soff, doff)
            assert (got[:doff] == 0xCD).all() and (got[doff + size:] == 0xCD).all()
            assert (rt.download(b, 0, (4096,), np.uint8) == 0xCD).all()
        note("host get of %d bytes" % size)
        rt.lib.nvshmemx_getmem_on_stream(rt.ptr(a, 1) + 7, b + 5, size, 2, s.ptr)   # PE 2's b -> PE 1's a
        s.synchronize()
        assert np.array_equal(rt.download(a, 1, (size,), np.uint8, 7), data[16:16 + size])
        host = np.zeros(size, np.uint8)                                             # pageable host memory
        rt.lib.nvshmemx_getmem_on_stream(host.ctypes.data_as(C.c_void_p), b + 5, size, 2, s.ptr)
        s.synchronize()
        assert np.array_equal(host, data[16:16 + size])
        s.destroy()
        rt.free(a); rt.free(b)
