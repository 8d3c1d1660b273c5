"""GPU parity of the host-initiated typed / sized / strided RMA forms and the typed waits on a
stream.  Expected values follow the operator definitions (strided forms: element i of the source
at stride sst goes to element i*dst of the destination)."""
import ctypes as C

import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import note, runtime
from nvshmem_amd import hip

pytestmark = pytest.mark.gpu
NPES = 4
vp, sz, pd, i32 = C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_int


def _fn(lib, name, restype, argtypes):
    f = getattr(lib, name)
    f.restype, f.argtypes = restype, argtypes
    return f


def test_host_typed_sized_strided_rma_and_waits():
    with runtime(NPES, 16 << 20) as rt:
        lib = rt.lib
        n = 4096
        a = rt.malloc(n); b = rt.malloc(n)
        A = O.fill_all("bytes", NPES, n, 55)
        rt.upload_all(a, A)
        s = hip.Stream()

        def reset():
            rt.fill(b, 0xEE, n)

        # sized put / get, blocking and on a stream
        reset()
        note("put64 / get16_on_stream / put128_nbi")
        _fn(lib, "nvshmem_put64", None, [vp, vp, sz, i32])(b, a, 5, 2)            # PE0.a -> PE2.b, 40 B
        assert np.array_equal(rt.download(b, 2, (40,), np.uint8), A[0, :40])
        _fn(lib, "nvshmemx_get16_on_stream", None, [vp, vp, sz, i32, vp])(b + 64, a + 64, 7, 3, s.ptr)
        _fn(lib, "nvshmemx_put128_nbi_on_stream", None, [vp, vp, sz, i32, vp])(b + 128, a + 128, 2, 1, s.ptr)
        s.synchronize()
        assert np.array_equal(rt.download(b, 0, (14,), np.uint8, 64), A[3, 64:78])
        assert np.array_equal(rt.download(b, 1, (32,), np.uint8, 128), A[0, 128:160])

        # strided: iput / iget, typed and sized
        reset()
        note("int32_iput / iget64_on_stream")
        _fn(lib, "nvshmem_int32_iput", None, [vp, vp, pd, pd, sz, i32])(b, a, 3, 2, 10, 1)
        got = rt.download(b, 1, (n,), np.uint8).view(np.int32)
        src = A[0].view(np.int32)
        want = np.full(n // 4, 0xEEEEEEEE, np.uint32).view(np.int32)
        for i in range(10):
            want[i * 3] = src[i * 2]
        assert np.array_equal(got, want)
        _fn(lib, "nvshmemx_iget64_on_stream", None, [vp, vp, pd, pd, sz, i32, vp])(b + 1024, a + 1024, 2, 5, 6, 3, s.ptr)
        s.synchronize()
        got = rt.download(b, 0, (n - 1024,), np.uint8, 1024).view(np.int64)
        src = A[3, 1024:].view(np.int64)
        for i in range(6):
            assert got[i * 2] == src[i * 5]
            assert got[i * 2 + 1] == np.int64(-0x1111111111111112)          # 0xEE.. untouched
        # a stride below 1 is refused
        _fn(lib, "nvshmem_iput8", None, [vp, vp, pd, pd, sz, i32])(b, a, 0, 1, 4, 1)
        assert b"stride" in lib.nvshmemx_amd_last_error()

        # scalar p / g
        note("float_p / int64_g / bfloat16 p,g")
        _fn(lib, "nvshmem_float_p", None, [vp, C.c_float, i32])(b + 2048, 3.25, 2)
        assert rt.download(b, 2, (1,), np.float32, 2048)[0] == np.float32(3.25)
        g = _fn(lib, "nvshmem_int64_g", C.c_int64, [vp, i32])
        assert g(a + 512, 3) == A[3, 512:520].view(np.int64)[0]
        _fn(lib, "nvshmemx_uint16_p_on_stream", None, [vp, C.c_uint16, i32, vp])(b + 2060, 0xBEEF, 1, s.ptr)
        s.synchronize()
        assert rt.download(b, 1, (1,), np.uint16, 2060)[0] == 0xBEEF
        gd = _fn(lib, "nvshmemx_double_g_on_stream", C.c_double, [vp, i32, vp])
        assert np.float64(gd(a + 256, 1, s.ptr)).view(np.int64) == A[1, 256:264].view(np.int64)[0]

        # typed put with signal on a stream, signal_fetch, typed waits
        note("double_put_signal_on_stream / signal_fetch / int_wait_until_on_stream")
        sig = rt.calloc(2, 8)
        _fn(lib, "nvshmemx_double_put_signal_on_stream", None,
            [vp, vp, sz, vp, C.c_uint64, i32, i32, vp])(b + 3000 + 8, a + 3000 + 8, 4, sig, 9, N.SIGNAL_ADD, 0, s.ptr)
        s.synchronize()
        assert _fn(lib, "nvshmem_signal_fetch", C.c_uint64, [vp])(sig) == 9
        assert np.array_equal(rt.download(b, 0, (32,), np.uint8, 3008), A[0, 3008:3040])
        flags = rt.calloc(4, 4)
        rt.upload(flags, 0, np.array([-5, 7, 7, 7], np.int32))
        status = rt.malloc(16)
        rt.upload(status, 0, np.array([1, 0, 0, 0], np.int32))          # element 0 is excluded
        _fn(lib, "nvshmemx_int_wait_until_on_stream", None, [vp, i32, i32, vp])(flags, N.CMP["LT"], 0, s.ptr)
        _fn(lib, "nvshmemx_int_wait_until_all_on_stream", None,
            [vp, sz, vp, i32, i32, vp])(flags, 4, status, N.CMP["EQ"], 7, s.ptr)
        _fn(lib, "nvshmemx_uint64_wait_until_on_stream", None, [vp, i32, C.c_uint64, vp])(sig, N.CMP["GE"], 9, s.ptr)
        s.synchronize()
        assert rt.read_timeout(0)[0] == 0
        # signed comparison is really signed: -5 < 0 held above; an unsigned type must not see it so
        rt.lib.nvshmemx_amd_set_spin_limit(100)
        _fn(lib, "nvshmemx_uint_wait_until_on_stream", None, [vp, i32, C.c_uint, vp])(flags, N.CMP["LT"], 5, s.ptr)
        s.synchronize()
        rt.lib.nvshmemx_amd_set_spin_limit(1 << 22)
        flag, rec = rt.read_timeout(0)
        assert flag >= 1 and rec[2] == 0xFFFFFFFB and rec[3] == 5      # found (uint)-5, expected 5
        s.destroy()


def test_wait_until_all_vector_on_stream():
    with runtime(NPES, 1 << 20) as rt:
        lib = rt.lib
        s = hip.Stream()
        flags = rt.calloc(4, 8); values = rt.malloc(32); status = rt.malloc(16)
        rt.upload(flags, 0, np.array([3, 10, -2, 99], np.int64))
        rt.upload(values, 0, np.array([3, 11, -2, 5], np.int64))       # element 1 does not match ...
        rt.upload(status, 0, np.array([0, 1, 0, 0], np.int32))         # ... and is excluded
        wait = _fn(lib, "nvshmemx_int64_wait_until_all_vector_on_stream", None, [vp, sz, vp, i32, vp, vp])
        note("int64 wait_until_all_vector_on_stream GE")
        wait(flags, 4, status, N.CMP["GE"], values, s.ptr)
        s.synchronize()
        assert rt.read_timeout(0)[0] == 0
        # more variables than one batch of polls: 21 of them, two excluded, all others satisfied ...
        many = rt.calloc(21, 8); mvals = rt.malloc(21 * 8); mstat = rt.malloc(21 * 4)
        have = np.arange(21, dtype=np.int64) * 3
        want = have.copy(); want[[4, 13]] += 1                          # 4 and 13 do not match ...
        st = np.zeros(21, np.int32); st[[4, 13]] = 1                    # ... and are excluded
        rt.upload(many, 0, have); rt.upload(mvals, 0, want); rt.upload(mstat, 0, st)
        wait(many, 21, mstat, N.CMP["EQ"], mvals, s.ptr)
        s.synchronize()
        assert rt.read_timeout(0)[0] == 0
        # without the exclusion the wait on element 1 runs into the spin limit and is recorded
        rt.lib.nvshmemx_amd_set_spin_limit(100)
        wait(flags, 4, None, N.CMP["GE"], values, s.ptr)
        s.synchronize()
        rt.lib.nvshmemx_amd_set_spin_limit(1 << 22)
        flag, rec = rt.read_timeout(0)
        assert flag >= 1 and rec[2] == 10 and rec[3] == 11
        # ... and with 13 in the set the wait gives up there, having passed the twelve in front of it
        st[13] = 0
        rt.upload(mstat, 0, st)
        rt.lib.nvshmemx_amd_set_spin_limit(100)
        wait(many, 21, mstat, N.CMP["EQ"], mvals, s.ptr)
        s.synchronize()
        rt.lib.nvshmemx_amd_set_spin_limit(1 << 22)
        flag, rec = rt.read_timeout(0)
        assert flag >= 1 and rec[2] == 39 and rec[3] == 40, rec
        assert rec[1] == rt.ptr(many, 0) + 13 * 8
        wait(flags, 4, None, 17, values, s.ptr)
        assert b"unknown comparison" in lib.nvshmemx_amd_last_error()
        wait(flags, 4, None, N.CMP["GE"], None, s.ptr)
        assert b"cmp_values is NULL" in lib.nvshmemx_amd_last_error()
        s.destroy()


AMO_BITWISE = [("uint", 32), ("ulong", 64), ("ulonglong", 64), ("int32", 32), ("int64", 64),
               ("uint32", 32), ("uint64", 64)]
AMO_STANDARD = AMO_BITWISE + [("int", 32), ("long", 64), ("longlong", 64), ("size", 64), ("ptrdiff", 64)]
SIGNED = {"int32", "int64", "int", "long", "longlong", "ptrdiff"}


def _ctype(name, bits):
    if name in ("float", "double"):
        return C.c_float if bits == 32 else C.c_double
    if name in SIGNED:
        return C.c_int32 if bits == 32 else C.c_int64
    return C.c_uint32 if bits == 32 else C.c_uint64


def test_host_atomics_every_name_against_the_oracle():
    """The blocking host forms apply the same operations as the device forms: compare the word left
    behind and the value returned with the oracle's integer model, on a remote PE."""
    rng = np.random.default_rng(77)
    with runtime(NPES, 1 << 20) as rt:
        lib = rt.lib
        word = rt.calloc(1, 8)
        count = 0

        def check(name, bits, op, cond_kind=None):
            nonlocal count
            ct = _ctype(name, bits)
            mask = 2**bits - 1
            pe = 1 + count % (NPES - 1)
            init = int(rng.integers(0, 2**64, dtype=np.uint64))
            value = int(rng.integers(0, 2**64, dtype=np.uint64))
            cond = (init & mask) if cond_kind == "hit" else ((init ^ 1) & mask)
            rt.upload(word, pe, np.array([init], np.uint64))
            fname = "nvshmem_" + name + "_atomic_" + op
            fetching = op in ("fetch", "swap", "compare_swap", "fetch_add", "fetch_inc", "fetch_and",
                              "fetch_or", "fetch_xor")
            args = {"fetch": [], "inc": [], "fetch_inc": [], "compare_swap": [ct, ct]}.get(op, [ct])
            f = _fn(lib, fname, ct if fetching else None, [vp] + args + [i32])

            def as_c(v):   # the low `bits` bits as a value of the C type
                v &= mask
                if ct in (C.c_int32, C.c_int64) and v >> (bits - 1):
                    v -= 1 << bits
                return v
            call = [word] + ([as_c(cond), as_c(value)] if op == "compare_swap" else [as_c(value)] * len(args)) + [pe]
            got = f(*call)
            new, fetched = O.amo(op, bits, init, value, cond)
            left = int(rt.download(word, pe, (1,), np.uint64)[0])
            assert left == (init & ~mask) | new, (fname, cond_kind, hex(init), hex(value))
            if fetching:
                assert (int(got) & mask) == fetched, (fname, cond_kind)
            count += 1

        for name, bits in AMO_STANDARD:
            for op in ("fetch", "set", "swap", "fetch_add", "add", "fetch_inc", "inc"):
                check(name, bits, op)
            check(name, bits, "compare_swap", "hit")
            check(name, bits, "compare_swap", "miss")
        for name, bits in AMO_BITWISE:
            for op in ("fetch_and", "and", "fetch_or", "or", "fetch_xor", "xor"):
                check(name, bits, op)
        assert count == 12 * 9 + 7 * 6
        # float / double: fetch, set, swap move the bits unchanged
        for name, ct, npt in (("float", C.c_float, np.float32), ("double", C.c_double, np.float64)):
            fword = rt.calloc(1, 8)
            amo_name = lambda op: "nvshmem_" + name + "_atomic_" + op
            _fn(lib, amo_name("set"), None, [vp, ct, i32])(fword, 1.5, 2)
            assert _fn(lib, amo_name("fetch"), ct, [vp, i32])(fword, 2) == 1.5
            assert _fn(lib, amo_name("swap"), ct, [vp, ct, i32])(fword, -0.25, 2) == 1.5
            assert rt.download(fword, 2, (1,), npt)[0] == npt(-0.25)
            assert rt.download(fword, 1, (1,), npt)[0] == 0
        # errors are reported, not executed
        f = _fn(lib, "nvshmem_int_atomic_fetch_add", C.c_int32, [vp, C.c_int32, i32])
        assert f(word, 1, NPES) == 0 and b"outside" in lib.nvshmemx_amd_last_error()
        assert f(word + 2, 1, 1) == 0 and b"aligned" in lib.nvshmemx_amd_last_error()
