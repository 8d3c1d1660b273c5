"""Size sweeps in the reference's perftest conventions, printed as tables.

    python3 nvshmem_amd/perftest_sweep.py [--what put,get,reduce,coll,moe] [--iters N]

put / get : message sizes 8 B .. 256 MiB (powers of two), 8 logical PEs, PE p -> (p+1)%8,
            1 / 4 / 16 blocks of 1024 threads per PE plus the "filled GPU" shape (one block of
            64 threads per 1 KiB).  Bandwidth counts the payload once, as perftest/device/pt-to-pt/shmem_put_bw.cu:268
            does, summed over the 8 PEs; latency is the launch-to-completion time of one exchange.
reduce    : config 3 (8 PEs x 2^26): fp32 sum/max, bf16 sum/max, int64 xor, and config 1.
coll      : config 4 (16 PEs x 2^22): fcollect and alltoall, fp32 and int64.
moe       : config 5 dispatch and combine.
Collective bandwidth is algorithmic bytes (each source byte read once, each destination byte
written once) per second.
"""
import argparse
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def timeit(fn, iters, warm, hip):
    for _ in range(warm):
        fn()
    hip.synchronize()
    e0, e1 = hip.Event(), hip.Event()
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    e1.synchronize()
    ms = e0.elapsed_ms(e1) / iters
    e0.destroy(); e1.destroy()
    return ms


def sweep_rma(N, hip, is_get, iters):
    npes = 8
    rt = N.Runtime(npes=npes, symmetric_size=(512 << 20) + (16 << 20))
    perf = rt.perftest()
    smax = 1 << 28
    src = rt.calloc(smax, 1); dst = rt.calloc(smax, 1)
    name = "get" if is_get else "put"
    print("\n%smem_block ring, %d logical PEs; payload GB/s summed over PEs (latency us)" % (name, npes))
    print("%12s %22s %22s %22s %22s" % ("bytes/PE", "1 block x1024", "4 blocks x1024", "16 blocks x1024",
                                        "1 KiB per block x64"))
    for p in range(3, 29):
        size = 1 << p
        cells = []
        for blocks, threads in ((1, 1024), (4, 1024), (16, 1024), (max(1, size >> 10), 64)):
            n = iters if size >= (1 << 20) else iters * 5
            ms = timeit(lambda: perf.nvshmem_perftest_ring_rma(dst, src, size, blocks, threads,
                                                               N.SCOPE_BLOCK, is_get, 1, None), n, 3, hip)
            cells.append("%10.1f (%8.1f)" % (npes * size / ms / 1e6, ms * 1e3))
        print("%12d %s" % (size, " ".join("%22s" % c for c in cells)))
    rt.finalize()


def sweep_reduce(N, hip, iters):
    from nvshmem_amd import _lib
    npes = 8
    n = 1 << 26
    rt = N.Runtime(npes=npes, symmetric_size=2 * n * 8 + (16 << 20))
    print("\nallreduce, %d logical PEs, fixed PE order; algorithmic GB/s = 2*npes*n*sizeof(T)/t" % npes)
    print("%-28s %12s %12s %10s" % ("call", "elements/PE", "GB/s", "ms"))
    src = rt.calloc(n, 8); dst = rt.calloc(n, 8)
    for t, op, es, cnt in (("int32", "sum", 4, 1 << 20), ("float", "sum", 4, n), ("float", "max", 4, n),
                           ("bfloat16", "sum", 2, n), ("bfloat16", "max", 2, n), ("int64", "xor", 8, n)):
        fn = _lib.typed_coll(rt.lib, "nvshmemx_%s_%s_reduce_on_stream" % (t, op), True)
        ms = timeit(lambda: fn(0, dst, src, cnt, None), iters, 3, hip)
        print("%-28s %12d %12.1f %10.4f" % ("%s_%s_reduce" % (t, op), cnt, 2 * npes * cnt * es / ms / 1e6, ms))
    rt.finalize()


def sweep_coll(N, hip, iters):
    npes, n = 16, 1 << 22
    print("\nfcollect / alltoall, %d logical PEs x 2^22 elements; algorithmic GB/s" % npes)
    print("%-28s %12s %10s" % ("call", "GB/s", "ms"))
    for t, es in (("float", 4), ("int64", 8)):
        rt = N.Runtime(npes=npes, symmetric_size=n * es * 18 + (16 << 20))
        src = rt.calloc(n, es); fdst = rt.calloc(16 * n, es); adst = rt.calloc(n, es)
        ms = timeit(lambda: rt.alltoall(t, adst, src, n // npes), iters, 3, hip)
        print("%-28s %12.1f %10.4f" % ("%s_alltoall" % t, 2 * npes * n * es / ms / 1e6, ms))
        ms = timeit(lambda: rt.fcollect(t, fdst, src, n), iters, 3, hip)
        print("%-28s %12.1f %10.4f" % ("%s_fcollect" % t, (npes + npes * npes) * n * es / ms / 1e6, ms))
        rt.finalize()


def sweep_moe(N, hip, iters):
    import numpy as np
    import oracle_lib as O
    npes, T, K, E, row = 8, 8192, 8, 256, 7168 * 2
    ex = O.moe_routing(npes, T, K, E, 1.1, 8)
    counts, _, dest_pe, dest_row, recv_rows = O.moe_plan(ex, npes, T, K, E)
    cap, rows = int(recv_rows.max()), T * K
    rt = N.Runtime(npes=npes, symmetric_size=cap * row + rows * row + T * row + (64 << 20))
    perf = rt.perftest()
    send = rt.calloc(T * row, 1); recv = rt.malloc(cap * row); out = rt.malloc(rows * row)
    d_pe = rt.malloc(rows * 4); d_row = rt.malloc(rows * 8)
    expected = rt.malloc(npes * 8); sig = rt.calloc(npes, 8)
    rt.upload_all(d_pe, dest_pe); rt.upload_all(d_row, dest_row)
    epp = E // npes
    rt.upload_all(expected, np.stack([[counts[s, d * epp:(d + 1) * epp].sum() for s in range(npes)]
                                      for d in range(npes)]).astype(np.uint64))
    def timed_dispatch(launch):
        best = None
        for _ in range(iters + 1):
            perf.nvshmem_perftest_fill_words(sig, 0, npes, None)
            hip.synchronize()
            e0, e1 = hip.Event(), hip.Event()
            e0.record()
            rc = launch()
            e1.record(); e1.synchronize()
            assert rc == 0
            ms = e0.elapsed_ms(e1)
            best = ms if best is None else min(best, ms)
        return best
    best = timed_dispatch(lambda: perf.nvshmem_perftest_moe_dispatch(recv, cap, send, d_pe, d_row, expected,
                                                                     sig, T, K, row, 32, 256, None))
    best_pieces = timed_dispatch(lambda: perf.nvshmem_perftest_moe_dispatch_pieces(
        recv, cap, send, d_pe, d_row, expected, sig, T, K, row, 1024, 256, None))
    moved = npes * rows * row
    print("\nMoE token shuffle, 8 PEs x 8192 tokens x 7168 bf16, top-8 of 256 experts, Zipf(1.1); "
          "busiest PE receives %d of %d rows" % (cap, npes * rows))
    print("dispatch (put + signal ADD + wait GE): %.3f ms; %.1f GB/s on the HBM lower bound "
          "(rows read once, written 8x = %.3f GiB); %.1f GB/s if every copy re-read its row"
          % (best, (moved + moved / K) / best / 1e6, (moved + moved / K) / 2**30, 2 * moved / best / 1e6))
    print("dispatch (1 KiB items stored through nvshmem_ptr, then signals): %.3f ms; %.1f GB/s on the lower bound"
          % (best_pieces, (moved + moved / K) / best_pieces / 1e6))
    ms = timeit(lambda: perf.nvshmem_perftest_moe_combine(out, recv, cap, d_pe, d_row, T, K, row, 8192, 256,
                                                          None), iters, 2, hip)
    print("combine  (getmem_nbi per copy):        %.3f ms; %.1f GB/s (%.3f GiB read + written)"
          % (ms, 2 * moved / ms / 1e6, 2 * moved / 2**30))
    ms = timeit(lambda: perf.nvshmem_perftest_moe_combine_pieces(out, recv, cap, d_pe, d_row, T, K, row, 2048,
                                                                 262144, 64, N.SCOPE_WARP, None), iters, 2, hip)
    print("combine  (getmem_nbi per 2 KiB piece):  %.3f ms; %.1f GB/s" % (ms, 2 * moved / ms / 1e6))
    assert all(rt.read_timeout(pe)[0] == 0 for pe in range(npes))
    rt.finalize()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--what", default="put,get,reduce,coll,moe")
    ap.add_argument("--iters", type=int, default=20)
    args = ap.parse_args()
    import nvshmem_amd as N
    from nvshmem_amd import hip
    what = args.what.split(",")
    if "put" in what:
        sweep_rma(N, hip, 0, args.iters)
    if "get" in what:
        sweep_rma(N, hip, 1, args.iters)
    if "reduce" in what:
        sweep_reduce(N, hip, args.iters)
    if "coll" in what:
        sweep_coll(N, hip, args.iters)
    if "moe" in what:
        sweep_moe(N, hip, max(3, args.iters // 4))


if __name__ == "__main__":
    main()
