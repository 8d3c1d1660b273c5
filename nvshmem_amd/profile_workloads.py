"""Runs the benchmark's kernels a few times each, for use under rocprofv3:

    rocprofv3 --kernel-trace --stats -d <out> -- python3 nvshmem_amd/profile_workloads.py
    rocprofv3 --pmc FETCH_SIZE -d <out> -- python3 nvshmem_amd/profile_workloads.py
    rocprofv3 --pmc WRITE_SIZE -d <out> -- python3 nvshmem_amd/profile_workloads.py

Workloads (same shapes as bench.py): plain_copy calibration (1 GiB read + 1 GiB written),
put_block (8 PEs x 256 MiB), float sum reduce (8 PEs x 2^26), float sum reducescatter (8 PEs, 256 MiB
source per PE), broadcast (8 PEs x 256 MiB), then with 16 PEs alltoall and fcollect (2^22 fp32 per
PE).  The large sources hold random data, as in bench.py: HBM moves all-zero buffers a few per
cent faster, and the durations here are meant to agree with the benchmark's.
"""
import argparse
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def moe_plan(np, rng, npes, tokens, topk, experts, zipf_s):
    """Routing and receive layout of the MoE shuffle: top-k distinct experts per token with
    P(expert k) ~ (k + 1)^-s (drawn without replacement through Gumbel keys), rows grouped on the
    destination PE by (expert, source PE, token order).  -> dest_pe, dest_row [npes, tokens * topk],
    expected [dst, src] row counts, rows received per PE."""
    logp = -zipf_s * np.log(np.arange(1, experts + 1))
    per_pe = experts // npes
    picks = np.empty((npes, tokens, topk), np.int64)
    for pe in range(npes):
        keys = logp[None, :] + rng.gumbel(size=(tokens, experts))
        picks[pe] = np.argsort(-keys, axis=1)[:, :topk]
    counts = np.stack([np.bincount(picks[pe].reshape(-1), minlength=experts) for pe in range(npes)])  # [src, expert]
    # segment (expert, src) starts after all segments in front of it on the expert's PE
    seg = np.zeros((experts, npes), np.int64)
    recv_rows = np.zeros(npes, np.int64)
    for d in range(npes):
        run = 0
        for e in range(d * per_pe, (d + 1) * per_pe):
            for src in range(npes):
                seg[e, src] = run
                run += counts[src, e]
        recv_rows[d] = run
    dest_pe = (picks // per_pe).reshape(npes, -1).astype(np.int32)
    dest_row = np.empty((npes, tokens * topk), np.int64)
    for pe in range(npes):
        flat = picks[pe].reshape(-1)
        order = np.argsort(flat, kind="stable")                       # copies of one expert in token order
        rank = np.empty_like(order)
        starts = np.concatenate(([0], np.cumsum(counts[pe])[:-1]))
        rank[order] = np.arange(flat.size) - starts[flat[order]]
        dest_row[pe] = seg[flat, pe] + rank
    expected = np.stack([[counts[src, d * per_pe:(d + 1) * per_pe].sum() for src in range(npes)]
                         for d in range(npes)]).astype(np.uint64)
    return dest_pe, dest_row, expected, recv_rows


def moe_shuffle(N, hip, np, rng, noise, iters):
    """Config 5: 8 PEs x 8192 tokens x 7168 bf16, top-8 of 256 experts, Zipf(1.1): dispatch, then combine."""
    npes, T, K, E, row = 8, 8192, 8, 256, 7168 * 2
    dest_pe, dest_row, expected, recv_rows = moe_plan(np, rng, npes, T, K, E, 1.1)
    cap, rows = int(recv_rows.max()), T * K
    rt = N.Runtime(npes=npes, symmetric_size=cap * row + rows * row + T * row + (64 << 20))
    perf = rt.perftest()
    send = rt.malloc(T * row); recv = rt.malloc(cap * row); out = rt.malloc(rows * row)
    d_pe = rt.malloc(rows * 4); d_row = rt.malloc(rows * 8)
    d_expected = rt.malloc(npes * 8); sig = rt.calloc(npes, 8)
    for pe in range(npes):
        rt.upload(send, pe, np.roll(noise[:T * row], 4096 * (pe + 1)))
    rt.upload_all(d_pe, dest_pe); rt.upload_all(d_row, dest_row); rt.upload_all(d_expected, expected)
    for _ in range(iters):
        assert perf.nvshmem_perftest_fill_words(sig, 0, npes, None) == 0
        assert perf.nvshmem_perftest_moe_dispatch_pieces(recv, cap, send, d_pe, d_row, d_expected, sig, T, K, row,
                                                         1024, 256, None) == 0
        assert perf.nvshmem_perftest_moe_combine_pieces(out, recv, cap, d_pe, d_row, T, K, row, 2048, 262144, 64,
                                                        N.SCOPE_WARP, None) == 0
    hip.synchronize()
    assert all(rt.read_timeout(pe)[0] == 0 for pe in range(npes)), "a receiver gave up waiting"
    # the round trip gives every row back: spot check
    for pe in (0, npes - 1):
        got = rt.download(out, pe, (64, row), np.uint8)
        want = np.repeat(np.roll(noise[:T * row], 4096 * (pe + 1)).reshape(T, row)[:8], K, axis=0)
        assert np.array_equal(got, want), "combine(dispatch(x)) != x"
    rt.finalize()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=10)
    args = ap.parse_args()
    import numpy as np
    import nvshmem_amd as N
    from nvshmem_amd import _lib, hip

    rng = np.random.default_rng(1)
    noise = rng.integers(0, 256, 1 << 28, dtype=np.uint8)     # 256 MiB, rotated per PE

    def randomize(rt, ptr, nbytes, as_float=False):
        for pe in range(rt.npes):
            block = np.roll(noise[:nbytes], 4096 * (pe + 1))
            if as_float:   # keep exponents small: random bit patterns would be NaN / inf heavy
                block = (block.view(np.uint32) & np.uint32(0x007FFFFF)) | np.uint32(0x3F800000)
                block = block.view(np.uint8)
            rt.upload(ptr, pe, block)

    # calibration copy: 1 GiB read, 1 GiB written
    rt = N.Runtime(npes=2, symmetric_size=(2 << 30) + (64 << 20))
    perf = rt.perftest()
    cal_a = rt.calloc(1 << 30, 1)
    cal_b = rt.calloc(1 << 30, 1)
    for _ in range(args.iters):
        assert perf.nvshmem_perftest_plain_copy(cal_b, cal_a, 1 << 30, None) == 0
    hip.synchronize()
    rt.finalize()

    # put_block: heap and buffer layout exactly as bench.py's bench_put_block
    S = 1 << 28
    rt = N.Runtime(npes=8, symmetric_size=2 * S + (64 << 20))
    src = rt.calloc(S, 1)
    dst = rt.calloc(S, 1)
    randomize(rt, src, S)
    for _ in range(args.iters):
        assert perf.nvshmem_perftest_ring_rma(dst, src, S, 262144, 64, N.SCOPE_BLOCK, 0, 1, None) == 0
    hip.synchronize()
    rt.finalize()

    # sum_reduce: as bench_sum_reduce
    n = 1 << 26
    rt = N.Runtime(npes=8, symmetric_size=2 * n * 4 + (64 << 20))
    src = rt.calloc(n, 4)
    dst = rt.calloc(n, 4)
    randomize(rt, src, n * 4, as_float=True)
    red = _lib.typed_coll(rt.lib, "nvshmemx_float_sum_reduce_on_stream", True)
    for _ in range(args.iters):
        assert red(N.TEAM_WORLD, dst, src, n, None) == 0
    hip.synchronize()
    rt.finalize()

    # reducescatter (source 8 blocks of 2^23 fp32 per PE) and broadcast (256 MiB from PE 3)
    n = 1 << 23
    rt = N.Runtime(npes=8, symmetric_size=9 * n * 4 + (64 << 20))
    src = rt.calloc(8 * n, 4)
    dst = rt.calloc(n, 4)
    randomize(rt, src, 8 * n * 4, as_float=True)
    for _ in range(args.iters):
        rt.reducescatter("float", "sum", dst, src, n, stream=None)
    hip.synchronize()
    rt.free(dst)
    dst = None
    rt.finalize()
    S = 1 << 28
    rt = N.Runtime(npes=8, symmetric_size=2 * S + (64 << 20))
    src = rt.calloc(S, 1)
    dst = rt.calloc(S, 1)
    randomize(rt, src, S)
    for _ in range(args.iters):
        rt.broadcastmem(dst, src, S, 3)
    hip.synchronize()
    rt.finalize()

    # alltoall as bench_alltoall, then fcollect of the same source into a 16x larger destination
    n = 1 << 22
    rt = N.Runtime(npes=16, symmetric_size=2 * n * 4 + (16 << 20))
    src = rt.calloc(n, 4)
    dst = rt.calloc(n, 4)
    randomize(rt, src, n * 4)
    for _ in range(args.iters):
        rt.alltoall("float", dst, src, n // 16, stream=None)
    hip.synchronize()
    rt.finalize()
    rt = N.Runtime(npes=16, symmetric_size=(512 << 20))
    src = rt.calloc(n, 4)
    dst = rt.calloc(16 * n, 4)
    randomize(rt, src, n * 4)
    for _ in range(args.iters):
        rt.fcollect("float", dst, src, n, stream=None)
    hip.synchronize()
    rt.finalize()
    moe_shuffle(N, hip, np, rng, noise, max(2, args.iters // 2))
    print("profile_workloads: done (%d iterations each)" % args.iters)


if __name__ == "__main__":
    main()
