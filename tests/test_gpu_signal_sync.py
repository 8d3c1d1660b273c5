"""GPU parity of signals, waits, scalar p/g and the in-kernel barrier (a5-a7) through the C ABI,
plus the reference's put_signal workloads (ping-pong, ring allreduce) with their known answers."""
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
    with runtime(NPES, 1 << 28) as r:
        yield r


def _words(rt, sym, n=1):
    return rt.download_all(sym, (n,), np.uint64)


def test_signal_add_accumulates_exactly_and_set_overwrites(rt):
    perf = rt.perftest()
    sig = rt.calloc(8, 8)
    L = O.lib()
    note("signal_op ADD")
    assert perf.nvshmem_perftest_signal_op(sig, 3, N.SIGNAL_ADD, 256, 10, None) == 0
    rt.sync()
    want = 0
    for _ in range(256 * 10):
        want = L.oracle_signal_op(want, 3, N.SIGNAL_ADD)
    assert (_words(rt, sig)[:, 0] == want).all() and want == 7680
    note("signal_op SET")
    assert perf.nvshmem_perftest_signal_op(sig, 41, N.SIGNAL_SET, 64, 2, None) == 0
    rt.sync()
    assert (_words(rt, sig)[:, 0] == L.oracle_signal_op(want, 41, N.SIGNAL_SET)).all()
    assert perf.nvshmem_perftest_signal_op(sig, 1, 7, 64, 1, None) != 0     # unknown operator
    rt.free(sig)


def test_host_signal_op_and_wait_on_stream(rt):
    sig = rt.calloc(8, 8)
    s = hip.Stream()
    note("signal_op_on_stream / signal_wait_until_on_stream")
    rt.lib.nvshmemx_signal_op_on_stream(sig, 5, N.SIGNAL_SET, 3, s.ptr)
    rt.lib.nvshmemx_signal_op_on_stream(sig, 2, N.SIGNAL_ADD, 3, s.ptr)
    rt.lib.nvshmemx_signal_op_on_stream(sig, 2, N.SIGNAL_ADD, 3, s.ptr)
    # the wait is stream-ordered behind the updates: it is satisfied when it starts
    rt.lib.nvshmemx_signal_wait_until_on_stream(rt.ptr(sig, 3), N.CMP["EQ"], 9, s.ptr)
    s.synchronize()
    w = _words(rt, sig)[:, 0]
    assert w[3] == 9 and w.sum() == 9
    assert rt.read_timeout(0)[0] == 0
    # put + signal from the host: data lands before the signal
    a = rt.malloc(4096); b = rt.calloc(4096, 1)
    data = O.fill_all("bytes", NPES, 4096, 21)
    rt.upload_all(a, data)
    rt.lib.nvshmemx_putmem_signal_on_stream(b, a, 4096, sig, 100, N.SIGNAL_SET, 6, s.ptr)
    s.synchronize()
    assert np.array_equal(rt.download(b, 6, (4096,), np.uint8), data[0])
    assert _words(rt, sig)[6, 0] == 100
    rt.lib.nvshmemx_signal_op_on_stream(sig, 1, 4, 0, s.ptr)
    assert b"neither SET" in rt.lib.nvshmemx_amd_last_error()
    s.destroy()
    rt.free(sig); rt.free(a); rt.free(b)


@pytest.mark.parametrize("cmp_name", ["EQ", "NE", "GT", "LE", "LT", "GE"])
def test_signal_wait_until_returns_the_satisfying_value(rt, cmp_name):
    perf = rt.perftest()
    L = O.lib()
    sig = rt.calloc(8, 8); out = rt.calloc(8, 8)
    # a preset value per PE that satisfies the comparison against 100 (checked with the oracle)
    preset = {"EQ": 100, "NE": 7, "GT": 101, "LE": 93, "LT": 3, "GE": 2**63}[cmp_name]
    assert L.oracle_compare_u64(preset, N.CMP[cmp_name], 100)
    for pe in range(NPES):
        rt.upload(sig, pe, np.array([preset + (0 if cmp_name == "EQ" else pe)], np.uint64))
    note("signal_wait_until cmp=%s" % cmp_name)
    assert perf.nvshmem_perftest_signal_wait(sig, N.CMP[cmp_name], 100, out, None) == 0
    rt.sync()
    got = _words(rt, out)[:, 0]
    for pe in range(NPES):
        assert got[pe] == preset + (0 if cmp_name == "EQ" else pe)
        assert rt.read_timeout(pe)[0] == 0
    rt.free(sig); rt.free(out)


def test_bounded_wait_gives_up_and_records_the_timeout(rt):
    # nobody ever signals: with a tiny poll limit the kernel must still finish, and the record says
    # which word was waited on, what was found and what was expected
    perf = rt.perftest()
    sig = rt.calloc(8, 8); out = rt.calloc(8, 8)
    rt.lib.nvshmemx_amd_set_spin_limit(200)
    try:
        note("bounded wait: spin limit 200, condition never true")
        before = rt.lib.nvshmemx_amd_timeout_count()
        assert perf.nvshmem_perftest_signal_wait(sig, N.CMP["GE"], 5, out, None) == 0
        rt.sync()
        # the host call that waited for the device reports the waits that gave up ...
        assert rt.lib.nvshmemx_amd_timeout_count() == before + NPES
        msg = rt.last_error()
        assert "%d device-side waits gave up" % NPES in msg and "spin limit of 200 polls" in msg
        # ... once: a second synchronisation has nothing new to say, a team barrier returns 0 again
        assert rt.lib.nvshmem_barrier(N.TEAM_WORLD) == 0
        assert perf.nvshmem_perftest_signal_wait(sig, N.CMP["GE"], 5, out, None) == 0
        assert rt.lib.nvshmem_barrier(N.TEAM_WORLD) != 0       # new timeouts: the barrier says so
        assert rt.lib.nvshmemx_amd_timeout_count() == before + 2 * NPES
        for pe in range(NPES):
            flag, rec = rt.read_timeout(pe)
            assert flag >= 1          # the number of this timeout in the GPU-wide count
            assert rec[1] == rt.ptr(sig, pe) and rec[2] == 0 and rec[3] == 5
            assert rt.read_timeout(pe)[0] == 0         # reading clears the record
    finally:
        rt.lib.nvshmemx_amd_set_spin_limit(1 << 22)
    rt.free(sig); rt.free(out)


def test_scalar_p_and_g(rt):
    perf = rt.perftest()
    words = rt.calloc(NPES, 8); out = rt.calloc(NPES, 8)
    note("uint64 p/g")
    assert perf.nvshmem_perftest_p_g(words, out, 1000, None) == 0
    rt.sync()
    w = rt.download_all(words, (NPES,), np.uint64)
    o = rt.download_all(out, (NPES,), np.uint64)
    for q in range(NPES):
        writer = (q - 1) % NPES
        assert w[q, writer] == 1000 + writer and w[q].sum() == 1000 + writer
        assert (o[:, q] == 1000 + writer).all()      # every PE read PE q's word with g
    rt.free(words); rt.free(out)


@pytest.mark.parametrize("scope,threads", [(N.SCOPE_THREAD, 1), (N.SCOPE_WARP, 64), (N.SCOPE_BLOCK, 256)])
def test_device_barrier_holds_every_pe(rt, scope, threads):
    perf = rt.perftest()
    counter = rt.calloc(1, 8); errors = rt.calloc(1, 8)
    note("barrier_all x200 scope=%d" % scope)
    assert perf.nvshmem_perftest_device_barrier(counter, errors, 200, scope, threads, None) == 0
    rt.sync()
    assert (_words(rt, errors)[:, 0] == 0).all()
    assert (_words(rt, counter)[:, 0] == 200).all()
    assert all(rt.read_timeout(pe)[0] == 0 for pe in range(NPES))
    rt.free(counter); rt.free(errors)


def test_put_signal_pingpong(rt):
    perf = rt.perftest()
    for nbytes in (8, 1000, 65536):
        data = rt.malloc(nbytes); sig = rt.calloc(1, 8)
        payload = O.fill_all("bytes", NPES, nbytes, 30)
        rt.upload_all(data, payload)
        note("put_signal ping-pong bytes=%d" % nbytes)
        assert perf.nvshmem_perftest_put_signal_pingpong(data, sig, nbytes, 50, 256, None) == 0
        rt.sync()
        got = rt.download_all(data, (nbytes,), np.uint8)
        assert np.array_equal(got[0], payload[0]) and np.array_equal(got[1], payload[0])
        assert np.array_equal(got[2:], payload[2:])          # bystanders untouched
        s = _words(rt, sig)[:, 0]
        assert s[0] == 50 and s[1] == 50 and (s[2:] == 0).all()
        assert all(rt.read_timeout(pe)[0] == 0 for pe in range(NPES))
        rt.free(data); rt.free(sig)


def test_fill_words_sets_every_pe_copy(rt):
    perf = rt.perftest()
    w = rt.malloc(1000 * 8)
    rt.fill(w, 0xAB, 1000 * 8)
    assert perf.nvshmem_perftest_fill_words(w + 8, 0x1122334455667788, 998, None) == 0
    rt.sync()
    got = rt.download_all(w, (1000,), np.uint64)
    assert (got[:, 1:999] == 0x1122334455667788).all()
    assert (got[:, 0] == 0xABABABABABABABAB).all() and (got[:, 999] == 0xABABABABABABABAB).all()
    rt.free(w)


def test_point_to_point_latency_loops_leave_the_documented_state(rt):
    # kinds of nvshmem_perftest_pt2pt_latency (include/nvshmem_perftest.h): what PE 0 and PE 1 hold
    # afterwards is fixed by the loop, so the timing kernels double as functional checks
    perf = rt.perftest()
    nbytes, iters = 4099, 37
    data = rt.malloc(nbytes); sig = rt.calloc(2, 8)
    payload = O.fill_all("bytes", NPES, nbytes, 31)

    def run(what, start=0):
        rt.upload_all(data, payload)
        rt.upload_all(sig, np.tile(np.array([start, 0], np.uint64), (NPES, 1)))
        note("pt2pt_latency kind=%d" % what)
        assert perf.nvshmem_perftest_pt2pt_latency(what, data, sig, nbytes, iters, 128, None) == 0
        rt.sync()
        assert all(rt.read_timeout(pe)[0] == 0 for pe in range(NPES))
        return rt.download_all(data, (nbytes,), np.uint8), _words(rt, sig, 2)

    got, w = run(0)                                            # put: PE 1 receives PE 0's bytes
    assert np.array_equal(got[1], payload[0]) and np.array_equal(got[0], payload[0])
    assert np.array_equal(got[2:], payload[2:]) and (w == 0).all()
    got, w = run(1)                                            # get: PE 0 fetches PE 1's bytes
    assert np.array_equal(got[0], payload[1]) and np.array_equal(got[1], payload[1])
    got, w = run(2)                                            # p: the last value written is iters
    assert w[1, 0] == iters and w[0, 0] == 0 and np.array_equal(got, payload)
    got, w = run(3, start=5)                                   # g: iters reads of the value 5
    assert w[0, 1] == 5 * iters and w[1, 0] == 5
    got, w = run(4, start=100)                                 # fetch_add chain on PE 1's word
    assert w[1, 0] == 100 + iters and w[0, 1] == 100 + iters - 1 and w[0, 0] == 100
    for what in (5, 6, 7):                                     # ping-pong: both words count the rounds
        got, w = run(what)
        assert w[0, 0] == iters and w[1, 0] == iters and (w[2:] == 0).all()
    assert perf.nvshmem_perftest_pt2pt_latency(8, data, sig, nbytes, iters, 128, None) != 0
    assert perf.nvshmem_perftest_pt2pt_latency(0, data, sig, nbytes, 0, 128, None) != 0
    rt.free(data); rt.free(sig)


def test_ring_allreduce_from_put_signal_known_answer_and_oracle(rt):
    perf = rt.perftest()
    blocks, chunk, chunks = 4, 1024, 3
    n = blocks * chunk * chunks
    dst = rt.calloc(n, 4); src = rt.malloc(n * 4); sig = rt.calloc(blocks, 8)
    # known answer of examples/ring-reduce.cu:209,242-248: src[i] = i on every PE -> dst[i] = i*npes
    rt.upload_all(src, np.tile(np.arange(n, dtype=np.int32), (NPES, 1)))
    note("ring_reduce known answer")
    assert perf.nvshmem_perftest_ring_reduce(dst, src, n, sig, chunk, blocks, 256, None) == 0
    rt.sync()
    got = rt.download_all(dst, (n,), np.int32)
    assert (got == np.arange(n, dtype=np.int32) * NPES).all()
    assert (_words(rt, sig, blocks) == 0).all()               # signals reset for the next run
    # seeded data against the oracle (integer sum: any order gives the same bits)
    data = O.fill_all("i32", NPES, n, 1)
    rt.upload_all(src, data)
    rt.fill(dst, 0, n * 4)
    note("ring_reduce seeded")
    assert perf.nvshmem_perftest_ring_reduce(dst, src, n, sig, chunk, blocks, 256, None) == 0
    rt.sync()
    got = rt.download_all(dst, (n,), np.int32)
    assert (got == O.reduce("i32", "sum", data)).all()
    assert all(rt.read_timeout(pe)[0] == 0 for pe in range(NPES))
    assert perf.nvshmem_perftest_ring_reduce(dst, src, n + 1, sig, chunk, blocks, 256, None) != 0
    rt.free(dst); rt.free(src); rt.free(sig)


PAYLOAD_ONLY = 0x100      # NVSHMEMX_AMD_SIGNAL_PAYLOAD_ONLY
SIGNAL_ADD = 10


@pytest.mark.parametrize("sig_op", [SIGNAL_ADD, SIGNAL_ADD | PAYLOAD_ONLY])
def test_put_signal_never_overtakes_its_payload(rt, sig_op):
    """Receivers read every message inside the kernel, straight after signal_wait_until returns: a
    signal that arrived ahead of its payload would leave words of an older message in the slot.  Both
    orderings of put-with-signal (the reference's full release and the payload-only hint), all three
    scopes, message sizes with and without the long-copy rounds, four PE pairs at once."""
    perf = rt.perftest()
    for scope, nbytes, slots, iters, blocks in ((N.SCOPE_BLOCK, 14336, 3, 200, 8), (N.SCOPE_BLOCK, 1 << 20, 2, 12, 4),
                                                (N.SCOPE_WARP, 14336, 4, 200, 16), (N.SCOPE_WARP, 40, 2, 300, 4),
                                                (N.SCOPE_WARP, 65536, 2, 40, 8), (N.SCOPE_THREAD, 256, 2, 50, 2)):
        data = rt.malloc(blocks * slots * nbytes); stage = rt.malloc(blocks * nbytes)
        sig = rt.calloc(2 * blocks, 8); errors = rt.calloc(1, 8)
        rt.fill(data, 0xFF, blocks * slots * nbytes)
        note("put_signal stream scope=%d bytes=%d slots=%d iters=%d blocks=%d sig_op=%#x"
             % (scope, nbytes, slots, iters, blocks, sig_op))
        assert perf.nvshmem_perftest_put_signal_stream(data, stage, sig, errors, nbytes, slots, iters, blocks,
                                                       scope, sig_op, None) == 0
        rt.sync()
        assert all(rt.read_timeout(pe)[0] == 0 for pe in range(NPES))
        assert (_words(rt, errors)[:, 0] == 0).all(), _words(rt, errors)[:, 0]
        s = _words(rt, sig, 2 * blocks).reshape(NPES, blocks, 2)
        assert (s[1::2, :, 0] == iters).all() and (s[0::2, :, 1] == iters).all()   # data counts, credits
        for p in (data, stage, sig, errors):
            rt.free(p)
    assert perf.nvshmem_perftest_put_signal_stream(0, 0, 0, 0, 12, 1, 1, 1, N.SCOPE_BLOCK, sig_op, None) != 0


def test_library_wide_put_signal_order(rt):
    """Call sites that pass plain NVSHMEM_SIGNAL_ADD, as code written for the reference does, get the
    payload-only order from the library option; the signal still never overtakes its payload, and the
    option goes back to the reference's order afterwards."""
    perf = rt.perftest()
    assert rt.lib.nvshmemx_amd_get_put_signal_order() == 0
    rt.lib.nvshmemx_amd_set_put_signal_order(1)
    try:
        assert rt.lib.nvshmemx_amd_get_put_signal_order() == 1
        for scope, nbytes, slots, iters, blocks in ((N.SCOPE_BLOCK, 14336, 3, 200, 8), (N.SCOPE_WARP, 14336, 4, 400, 16),
                                                    (N.SCOPE_THREAD, 256, 2, 50, 2)):
            data = rt.malloc(blocks * slots * nbytes); stage = rt.malloc(blocks * nbytes)
            sig = rt.calloc(2 * blocks, 8); errors = rt.calloc(1, 8)
            rt.fill(data, 0xFF, blocks * slots * nbytes)
            note("library-wide payload order: put_signal stream scope=%d bytes=%d" % (scope, nbytes))
            assert perf.nvshmem_perftest_put_signal_stream(data, stage, sig, errors, nbytes, slots, iters, blocks,
                                                           scope, SIGNAL_ADD, None) == 0
            rt.sync()
            assert all(rt.read_timeout(pe)[0] == 0 for pe in range(NPES))
            assert (_words(rt, errors)[:, 0] == 0).all(), _words(rt, errors)[:, 0]
            for p in (data, stage, sig, errors):
                rt.free(p)
    finally:
        rt.lib.nvshmemx_amd_set_put_signal_order(0)
    assert rt.lib.nvshmemx_amd_get_put_signal_order() == 0


def test_collective_launch_refuses_grids_that_cannot_be_co_resident(rt):
    perf = rt.perftest()
    dst = rt.calloc(1 << 20, 4); src = rt.calloc(1 << 20, 4); sig = rt.calloc(65535, 8)
    rc = perf.nvshmem_perftest_ring_reduce(dst, src, 65535 * 16, sig, 16, 65535, 1024, None)
    assert rc == 6      # NVSHMEMX_ERROR_COLLECTIVE_LAUNCH_FAILED
    assert b"co-resident" in rt.lib.nvshmemx_amd_last_error()
    rt.free(dst); rt.free(src); rt.free(sig)
