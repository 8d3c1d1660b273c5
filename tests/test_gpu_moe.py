"""GPU parity of the MoE token shuffle (a13): offsets exchange, dispatch with put + signal +
signal_wait_until, combine.  Bit-exact against the oracle's model."""
import numpy as np
import pytest

import nvshmem_amd as N
import oracle_lib as O
from gpu_util import note, runtime

pytestmark = pytest.mark.gpu


def _shuffle(rt, npes, T, K, E, row_bytes, blocks, threads, scope, seed_route=8, seed_data=7,
             check_exchange=True):
    perf = rt.perftest()
    ex = O.moe_routing(npes, T, K, E, 1.1, seed_route)
    counts, seg_base, dest_pe, dest_row, recv_rows = O.moe_plan(ex, npes, T, K, E)
    cap = int(recv_rows.max())
    rows = T * K
    send = rt.malloc(T * row_bytes)
    recv = rt.malloc(cap * row_bytes)
    out = rt.malloc(rows * row_bytes)
    d_pe = rt.malloc(rows * 4); d_row = rt.malloc(rows * 8)
    expected = rt.malloc(npes * 8); sig = rt.calloc(npes, 8)
    d_counts = rt.malloc(E * 8); d_seg = rt.malloc(E * npes * 8); d_recv_rows = rt.malloc(8)

    payload = np.stack([O.fill("bytes", T * row_bytes, seed_data, pe).reshape(T, row_bytes)
                        for pe in range(npes)])
    rt.upload_all(send, payload)
    rt.upload_all(d_pe, dest_pe)
    rt.upload_all(d_row, dest_row)
    # expected[dst][src] = rows src sends to dst
    epp = E // npes
    exp_tab = np.stack([[counts[src, d * epp:(d + 1) * epp].sum() for src in range(npes)]
                        for d in range(npes)]).astype(np.uint64)
    rt.upload_all(expected, exp_tab)
    rt.fill(recv, 0, cap * row_bytes)

    if check_exchange:
        rt.upload_all(d_counts, counts)
        note("moe_exchange_offsets E=%d" % E)
        assert perf.nvshmem_perftest_moe_exchange_offsets(d_counts, d_seg, d_recv_rows, E, None) == 0
        rt.sync()
        got_seg = rt.download_all(d_seg, (E, npes), np.int64)
        for pe in range(npes):
            assert np.array_equal(got_seg[pe], seg_base), pe
        assert np.array_equal(rt.download_all(d_recv_rows, (1,), np.int64)[:, 0], recv_rows)

    note("moe_dispatch T=%d K=%d row=%d blocks=%d threads=%d scope=%d" % (T, K, row_bytes, blocks, threads, scope))
    assert perf.nvshmem_perftest_moe_dispatch_ex(recv, cap, send, d_pe, d_row, expected, sig, T, K,
                                                 row_bytes, blocks, threads, scope, None) == 0
    rt.sync()
    assert all(rt.read_timeout(pe)[0] == 0 for pe in range(npes)), "a receiver gave up waiting"
    want_recv = O.moe_dispatch(payload, dest_pe, dest_row, recv_rows, T, K)
    for pe in range(npes):
        got = rt.download(recv, pe, (int(recv_rows[pe]), row_bytes), np.uint8)
        assert np.array_equal(got, want_recv[pe]), pe
    sigs = rt.download_all(sig, (npes,), np.uint64)
    assert np.array_equal(sigs, exp_tab)                 # ADD signals count the rows exactly

    # dispatch cut into short work items (two launches: data, then signals): same result, same signals.
    # Aligned buffers and rows take the load-once path, anything else the put path.
    for piece, threads in ((1024, 64), (2048, 128), (4096, 256)):
        rt.fill(recv, 0, cap * row_bytes)
        rt.fill(sig, 0, npes * 8)
        note("moe_dispatch_pieces piece=%d threads=%d row=%d" % (piece, threads, row_bytes))
        assert perf.nvshmem_perftest_moe_dispatch_pieces(recv, cap, send, d_pe, d_row, expected, sig, T, K,
                                                         row_bytes, piece, threads, None) == 0
        rt.sync()
        assert all(rt.read_timeout(pe)[0] == 0 for pe in range(npes)), "a receiver gave up waiting"
        for pe in range(npes):
            got = rt.download(recv, pe, (int(recv_rows[pe]), row_bytes), np.uint8)
            assert np.array_equal(got, want_recv[pe]), (piece, pe)
        assert np.array_equal(rt.download_all(sig, (npes,), np.uint64), exp_tab)
    assert perf.nvshmem_perftest_moe_dispatch_pieces(recv, cap, send, d_pe, d_row, expected, sig, T, K,
                                                     row_bytes, 512, 64, None) != 0
    assert perf.nvshmem_perftest_moe_dispatch_pieces(recv, cap, send, d_pe, d_row, expected, sig, T, K,
                                                     row_bytes, 1024, 96, None) != 0

    note("moe_combine")
    assert perf.nvshmem_perftest_moe_combine_ex(out, recv, cap, d_pe, d_row, T, K, row_bytes, blocks,
                                                threads, scope & 255, None) == 0
    rt.sync()
    want_out = O.moe_combine(want_recv, dest_pe, dest_row, T, K, row_bytes)
    for pe in range(npes):
        got = rt.download(out, pe, (rows, row_bytes), np.uint8)
        assert np.array_equal(got, want_out[pe]), pe
        assert np.array_equal(got, np.repeat(payload[pe], K, axis=0))   # round trip identity
    # the same with a work item of part of a row per wavefront (ragged last piece included)
    for piece in (1024, 2048, 4096):
        rt.fill(out, 0xEE, rows * row_bytes)
        note("moe_combine pieces of %d" % piece)
        assert perf.nvshmem_perftest_moe_combine_pieces(out, recv, cap, d_pe, d_row, T, K, row_bytes, piece,
                                                        4 * blocks, 64, N.SCOPE_WARP, None) == 0
        rt.sync()
        for pe in (0, npes - 1):
            assert np.array_equal(rt.download(out, pe, (rows, row_bytes), np.uint8), want_out[pe]), (piece, pe)
    assert perf.nvshmem_perftest_moe_combine_pieces(out, recv, cap, d_pe, d_row, T, K, row_bytes, 512,
                                                    blocks, 64, N.SCOPE_WARP, None) != 0
    for p in (send, recv, out, d_pe, d_row, expected, sig, d_counts, d_seg, d_recv_rows):
        rt.free(p)


@pytest.mark.parametrize("scope", [N.SCOPE_WARP, N.SCOPE_BLOCK, N.SCOPE_WARP | 256, N.SCOPE_BLOCK | 256])
def test_moe_shuffle_small(scope):
    with runtime(8, 1 << 28) as rt:
        _shuffle(rt, 8, 256, 8, 256, 1024, 4, 256, scope)
        _shuffle(rt, 8, 33, 3, 64, 200 + 6, 2, 128, scope, check_exchange=False)   # ragged rows


def test_moe_dispatch_pieces_through_the_put_api(monkeypatch):
    """NVSHMEM_PERFTEST_MOE_PUTS selects the nvshmemx_putmem_nbi_warp form of the short work items also
    for aligned rows (without it only rows that are not 16-byte aligned take it)."""
    monkeypatch.setenv("NVSHMEM_PERFTEST_MOE_PUTS", "1")
    with runtime(8, 1 << 28) as rt:
        _shuffle(rt, 8, 128, 8, 64, 4096 + 1024, 4, 256, N.SCOPE_WARP, check_exchange=False)


def test_moe_routing_table_outside_the_buffer_is_skipped_not_written():
    with runtime(4, 1 << 24) as rt:
        perf = rt.perftest()
        T, K, row = 16, 2, 64
        send = rt.calloc(T * row, 1); recv = rt.calloc(8 * row, 1)
        d_pe = rt.malloc(T * K * 4); d_row = rt.malloc(T * K * 8)
        expected = rt.calloc(4, 8); sig = rt.calloc(4, 8)
        bad_pe = np.full((4, T * K), 9, np.int32)          # PE 9 does not exist
        bad_row = np.full((4, T * K), 1 << 40, np.int64)   # far outside
        rt.upload_all(d_pe, bad_pe); rt.upload_all(d_row, bad_row)
        note("moe_dispatch with invalid routing entries")
        assert perf.nvshmem_perftest_moe_dispatch(recv, 8, send, d_pe, d_row, expected, sig, T, K,
                                                  row, 2, 128, None) == 0
        rt.sync()
        assert (rt.download_all(sig, (4,), np.uint64) == 0).all()
        note("moe_dispatch_pieces with invalid routing entries")
        assert perf.nvshmem_perftest_moe_dispatch_pieces(recv, 8, send, d_pe, d_row, expected, sig, T, K,
                                                         row, 1024, 128, None) == 0
        rt.sync()
        assert (rt.download_all(sig, (4,), np.uint64) == 0).all()
        assert (rt.download_all(recv, (8 * row,), np.uint8) == 0).all()


def test_config5_full_size_moe_shuffle():
    # 8 PEs x 8192 tokens x 7168 bf16, top-8 of 256 experts, Zipf(1.1): the receive buffer of the
    # busiest PE decides the symmetric allocation
    npes, T, K, E, row = 8, 8192, 8, 256, 7168 * 2
    ex = O.moe_routing(npes, T, K, E, 1.1, 8)
    recv_rows = O.moe_plan(ex, npes, T, K, E)[4]
    need = int(recv_rows.max()) * row + T * K * row + T * row + (64 << 20)
    with runtime(npes, need) as rt:
        _shuffle(rt, npes, T, K, E, row, 64, 256, N.SCOPE_WARP, check_exchange=True)


@pytest.mark.parametrize("scope,blocks,threads", [(N.SCOPE_WARP | 256 | 512, 64, 256), (N.SCOPE_BLOCK | 256 | 512, 128, 256),
                                                   (N.SCOPE_WARP | 256, 64, 256)])
def test_config5_full_size_dispatch_through_per_row_put_signal(scope, blocks, threads):
    """Config 5 at full size with one nvshmemx_putmem_signal_nbi per row copy (ADD 1 on the signal word of
    the source at the destination) and nvshmem_signal_wait_until(GE) on the receiver: every PE's receive
    buffer bit-exact against the oracle, signal counts exact.  Signal words sit on separate 128-byte
    lines (stride 16).  Payload-only ordering in both scopes, the reference's ordering once."""
    npes, T, K, E, row = 8, 8192, 8, 256, 7168 * 2
    ex = O.moe_routing(npes, T, K, E, 1.1, 8)
    counts, _, dest_pe, dest_row, recv_rows = O.moe_plan(ex, npes, T, K, E)
    cap, rows, stride = int(recv_rows.max()), T * K, 16
    with runtime(npes, cap * row + T * row + (64 << 20)) as rt:
        perf = rt.perftest()
        send = rt.malloc(T * row); recv = rt.malloc(cap * row)
        d_pe = rt.malloc(rows * 4); d_row = rt.malloc(rows * 8)
        expected = rt.malloc(npes * 8); sig = rt.calloc(npes * stride, 8)
        payload = np.stack([O.fill("bytes", T * row, 7, pe).reshape(T, row) for pe in range(npes)])
        rt.upload_all(send, payload); rt.upload_all(d_pe, dest_pe); rt.upload_all(d_row, dest_row)
        epp = E // npes
        exp_tab = np.stack([[counts[src, d * epp:(d + 1) * epp].sum() for src in range(npes)]
                            for d in range(npes)]).astype(np.uint64)
        rt.upload_all(expected, exp_tab)
        rt.fill(recv, 0, cap * row)
        note("moe_dispatch_put_signal full size scope=%#x blocks=%d threads=%d" % (scope, blocks, threads))
        assert perf.nvshmem_perftest_moe_dispatch_put_signal(recv, cap, send, d_pe, d_row, expected, sig, stride,
                                                             T, K, row, blocks, threads, scope, None) == 0
        rt.sync()
        assert all(rt.read_timeout(pe)[0] == 0 for pe in range(npes)), "a receiver gave up waiting"
        want_recv = O.moe_dispatch(payload, dest_pe, dest_row, recv_rows, T, K)
        for pe in range(npes):
            got = rt.download(recv, pe, (int(recv_rows[pe]), row), np.uint8)
            assert np.array_equal(got, want_recv[pe]), pe
        sigs = rt.download_all(sig, (npes * stride,), np.uint64).reshape(npes, npes, stride)
        assert np.array_equal(sigs[:, :, 0], exp_tab) and (sigs[:, :, 1:] == 0).all()
        # argument checks
        assert perf.nvshmem_perftest_moe_dispatch_put_signal(recv, cap, send, d_pe, d_row, expected, sig, 0,
                                                             T, K, row, blocks, threads, scope, None) != 0
        assert perf.nvshmem_perftest_moe_dispatch_put_signal(recv, cap, send, d_pe, d_row, expected, sig, 2,
                                                             T, K, row, 32, 256, N.SCOPE_WARP, None) != 0
        for p in (send, recv, d_pe, d_row, expected, sig):
            rt.free(p)
