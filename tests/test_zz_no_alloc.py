"""The dispatch entry point that allocates nothing (its signal words are a static device array of the
library) against the entry point it is a variant of, through the C ABI: same receive buffers, bit for
bit, on two calls in a row, the second with a smaller input."""
import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import note, runtime

pytestmark = pytest.mark.gpu


def _plan(npes, T, K, E, seed):
    ex = O.moe_routing(npes, T, K, E, 1.1, seed)
    counts, _, dest_pe, dest_row, recv_rows = O.moe_plan(ex, npes, T, K, E)
    epp = E // npes
    exp_tab = np.stack([[counts[src, d * epp:(d + 1) * epp].sum() for src in range(npes)]
                        for d in range(npes)]).astype(np.uint64)
    return dest_pe, dest_row, recv_rows, exp_tab


def test_static_dispatch_matches_the_dispatch_with_caller_signal_words():
    npes, K, E, row = 8, 8, 64, 4096 + 1024
    calls = ((512, 21, 1024, 128), (96, 22, 2048, 64))        # (tokens, routing seed, piece bytes, threads)
    cap = max(int(_plan(npes, T, K, E, seed)[2].max()) for T, seed, _, _ in calls)
    Tmax = max(c[0] for c in calls)
    with runtime(npes, 2 * cap * row + Tmax * row + (32 << 20)) as rt:
        perf = rt.perftest()
        assert perf.nvshmem_perftest_static_init() == 0      # the address of the static words, looked up up front
        send = rt.malloc(Tmax * row); recv_a = rt.malloc(cap * row); recv_b = rt.malloc(cap * row)
        d_pe = rt.malloc(Tmax * K * 4); d_row = rt.malloc(Tmax * K * 8)
        expected = rt.malloc(npes * 8); sig = rt.calloc(npes, 8)
        for T, seed, piece, threads in calls:
            dest_pe, dest_row, recv_rows, exp_tab = _plan(npes, T, K, E, seed)
            payload = np.stack([O.fill("bytes", T * row, 40 + seed, pe).reshape(T, row) for pe in range(npes)])
            rt.upload_all(send, payload); rt.upload_all(d_pe, dest_pe); rt.upload_all(d_row, dest_row)
            rt.upload_all(expected, exp_tab)
            rt.fill(recv_a, 0x5A, cap * row); rt.fill(recv_b, 0x5A, cap * row); rt.fill(sig, 0, npes * 8)
            note("moe_dispatch_pieces T=%d piece=%d" % (T, piece))
            assert perf.nvshmem_perftest_moe_dispatch_pieces(recv_a, cap, send, d_pe, d_row, expected, sig, T, K,
                                                             row, piece, threads, None) == 0
            note("moe_dispatch_pieces_static T=%d piece=%d" % (T, piece))
            assert perf.nvshmem_perftest_moe_dispatch_pieces_static(recv_b, cap, send, d_pe, d_row, expected, T, K,
                                                                    row, piece, threads, None) == 0
            rt.sync()
            assert all(rt.read_timeout(pe)[0] == 0 for pe in range(npes)), "a receiver gave up waiting"
            want = O.moe_dispatch(payload, dest_pe, dest_row, recv_rows, T, K)
            for pe in range(npes):
                a = rt.download(recv_a, pe, (cap, row), np.uint8)
                b = rt.download(recv_b, pe, (cap, row), np.uint8)
                assert np.array_equal(a, b), pe                               # the two entry points agree
                assert np.array_equal(b[:int(recv_rows[pe])], want[pe]), pe   # and with the oracle
                assert (b[int(recv_rows[pe]):] == 0x5A).all(), pe             # nothing else was written
        # bad arguments are refused like in the entry point it is a variant of
        assert perf.nvshmem_perftest_moe_dispatch_pieces_static(recv_b, cap, send, d_pe, d_row, expected, 16, K,
                                                                row, 512, 64, None) != 0
        for p in (send, recv_a, recv_b, d_pe, d_row, expected, sig):
            rt.free(p)


def test_static_dispatch_refuses_more_pes_than_its_signal_words_hold():
    with runtime(33, 1 << 20) as rt:
        perf = rt.perftest()
        x = rt.calloc(4096, 1)
        note("moe_dispatch_pieces_static with 33 PEs")
        assert perf.nvshmem_perftest_moe_dispatch_pieces_static(x, 1, x, x, x, x, 1, 1, 64, 1024, 64, None) != 0
        rt.free(x)
