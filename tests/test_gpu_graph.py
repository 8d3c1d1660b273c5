"""The on-stream collectives can be captured into a HIP graph: every replay (with fresh inputs and
eager work in between) must give what the eager calls give."""
import numpy as np
import pytest

import oracle_lib as O
from gpu_util import bits_equal, note, runtime
from nvshmem_amd import hip

pytestmark = pytest.mark.gpu


def test_graph_replays_match_eager_results():
    npes, n, seg = 8, 50021, 4099
    rng = np.random.default_rng(17)
    with runtime(npes, 64 << 20) as rt:
        src = rt.malloc(n * 4); red = rt.malloc(n * 4)
        a2a_src = rt.malloc(npes * seg); a2a_dst = rt.malloc(npes * seg); fc_dst = rt.malloc(npes * seg)
        s = hip.Stream()
        note("capturing reduce + alltoall + fcollect + signal_op into a graph")
        sig = rt.calloc(1, 8)
        with hip.Graph(s) as g:
            rt.reduce("float", "sum", red, src, n, stream=s)
            rt.alltoallmem(a2a_dst, a2a_src, seg, stream=s)
            rt.fcollectmem(fc_dst, a2a_src, seg, stream=s)
            rt.lib.nvshmemx_signal_op_on_stream(sig, 1, 10, 2, s.ptr)      # ADD 1 on PE 2
        for replay in range(4):
            f = rng.standard_normal((npes, n)).astype(np.float32)
            blocks = rng.integers(0, 256, (npes, npes * seg), dtype=np.uint8)
            rt.upload_all(src, f)
            rt.upload_all(a2a_src, blocks)
            rt.fill(red, 0xFF, n * 4); rt.fill(a2a_dst, 0xFF, npes * seg); rt.fill(fc_dst, 0xFF, npes * seg)
            note("graph replay %d" % replay)
            g.launch()
            s.synchronize()
            want = O.reduce("f32", "sum", f)
            for pe in (0, 7):
                assert bits_equal(rt.download(red, pe, (n,), np.float32), want), (replay, pe)
            assert np.array_equal(rt.download_all(a2a_dst, (npes * seg,), np.uint8), O.alltoall(blocks))
            assert np.array_equal(rt.download_all(fc_dst, (npes * seg,), np.uint8), O.fcollect(blocks[:, :seg]))
            assert rt.download(sig, 2, (1,), np.uint64)[0] == replay + 1
            # eager work between replays
            rt.reduce("float", "max", red, src, n)
            assert bits_equal(rt.download(red, 3, (n,), np.float32), O.reduce("f32", "max", f))
        g.destroy(); s.destroy()


def test_graph_with_team_collectives_broadcast_and_reducescatter():
    npes, n = 8, 4100
    rng = np.random.default_rng(18)
    with runtime(npes, 16 << 20) as rt:
        src = rt.malloc(npes * n * 4); rs = rt.malloc(n * 4); bc = rt.malloc(n * 4); row = rt.malloc(n * 4)
        x, y = rt.team_split_2d(0, 4)          # rows {0..3}, {4..7}; columns {p, p+4}
        s = hip.Stream()
        note("capturing reducescatter + broadcast + a reduce on every row of a 2-D split")
        with hip.Graph(s) as g:
            rt.reducescatter("float", "sum", rs, src, n, stream=s)
            rt.broadcastmem(bc, src, n * 4, 5, stream=s)
            rt.reduce("float", "sum", row, src, n, stream=s, team=x)
        for replay in range(3):
            f = rng.standard_normal((npes, npes * n)).astype(np.float32)
            rt.upload_all(src, f)
            for p in (rs, bc, row):
                rt.fill(p, 0xFF, n * 4)
            note("graph replay %d" % replay)
            g.launch()
            s.synchronize()
            assert bits_equal(rt.download_all(rs, (n,), np.float32), O.reducescatter("f32", "sum", f))
            got = rt.download_all(bc, (n,), np.float32)
            assert all(bits_equal(got[pe], f[5, :n]) for pe in range(npes))
            got = rt.download_all(row, (n,), np.float32)
            for lo in (0, 4):
                want = O.reduce("f32", "sum", f[lo:lo + 4, :n])
                assert all(bits_equal(got[pe], want) for pe in range(lo, lo + 4))
            rt.fcollectmem(src, bc, 64, team=y)     # eager work between replays
        g.destroy(); s.destroy()
        rt.team_destroy(x); rt.team_destroy(y)
