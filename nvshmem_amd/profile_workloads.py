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
    print("profile_workloads: done (%d iterations each)" % args.iters)


if __name__ == "__main__":
    main()
