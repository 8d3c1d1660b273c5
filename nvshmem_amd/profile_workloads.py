"""Runs the benchmark's workloads a few times each, for use under rocprofv3:

    rocprofv3 --kernel-trace --stats -d <out> -- python3 nvshmem_amd/profile_workloads.py
    rocprofv3 --pmc FETCH_SIZE -d <out> -- python3 nvshmem_amd/profile_workloads.py --iters 3
    rocprofv3 --pmc WRITE_SIZE -d <out> -- python3 nvshmem_amd/profile_workloads.py --iters 3
    (any other counter set the same way, one rocprofv3 run per set)

The workloads are the objects of nvshmem_amd/workloads.py, the ones bench.py times, with numpy noise as
input (the oracle is not involved).  Every workload is bracketed by two launches of the empty kernel
profile_marker_kernel, and the order of the workloads is written to --manifest, so that
nvshmem_amd/profile_summary.py can cut the trace into workloads by counting markers.  The first
workload is the counter calibration: a plain copy kernel that reads 1 GiB and writes 1 GiB.
"""
import argparse
import tempfile
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def noise_plan(np, rng, npes, tokens, topk, experts, zipf_s):
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--only", default="", help="comma-separated workload names")
    ap.add_argument("--manifest", default=os.path.join(tempfile.gettempdir(), "nvshmem_amd_profile_manifest.json"))
    args = ap.parse_args()
    import numpy as np
    import nvshmem_amd as N
    from nvshmem_amd import hip, workloads

    rng = np.random.default_rng(1)
    noise = rng.integers(0, 256, 1 << 28, dtype=np.uint8)     # 256 MiB, rotated per PE and tiled when short

    def gen(kind, npes, n, seed):
        """Noise of the right shape; floating-point kinds get bounded exponents (random bit patterns
        would be mostly NaN and infinity)."""
        dtype, es = {"bytes": (np.uint8, 1), "u64": (np.uint64, 8), "i32": (np.int32, 4), "f32": (np.float32, 4),
                     "bf16": (np.uint16, 2)}[kind]
        out = np.empty((npes, n * es), np.uint8)
        for pe in range(npes):
            row = np.roll(noise, 4096 * (pe + 1) + 64 * seed)
            reps = -(-n * es // row.size)
            out[pe] = np.tile(row, reps)[:n * es] if reps > 1 else row[:n * es]
        if kind == "f32":
            v = out.view(np.uint32)
            v &= np.uint32(0x807FFFFF); v |= np.uint32(0x3F800000)
        elif kind == "bf16":
            v = out.view(np.uint16)
            v &= np.uint16(0x807F); v |= np.uint16(0x3F80)
        return out.view(dtype)

    only = set(x for x in args.only.split(",") if x)
    manifest = []

    def bracket(perf, name, fn, iters):
        assert perf.nvshmem_perftest_profile_marker(None) == 0
        for _ in range(iters):
            fn()
        assert perf.nvshmem_perftest_profile_marker(None) == 0
        hip.synchronize()
        manifest.append({"name": name, "launches": iters})

    # counter calibration: 1 GiB read, 1 GiB written
    rt = N.Runtime(npes=2, symmetric_size=(2 << 30) + (64 << 20))
    perf = rt.perftest()
    cal_a = rt.calloc(1 << 30, 1)
    cal_b = rt.calloc(1 << 30, 1)

    def calibrate():
        assert perf.nvshmem_perftest_plain_copy(cal_b, cal_a, 1 << 30, None) == 0
    bracket(perf, "calibration", calibrate, args.iters)
    rt.finalize()

    plan = noise_plan(np, rng, 8, 8192, 8, 256, 1.1)
    for g in workloads.all_groups(plan) + workloads.profile_only_groups():
        if only and not any(n in only for n in g.names()):
            continue
        rt = N.Runtime(npes=g.npes, symmetric_size=g.heap_bytes)
        try:
            for item in g.setup(rt, gen):
                if only and item.name not in only:
                    continue
                if hasattr(item, "prepare"):
                    item.prepare()
                iters = max(2, args.iters // item.scale)
                item.step()                    # one untimed pass (first touch of the destination)
                hip.synchronize()
                bracket(rt.perftest(), item.name, item.step, iters)
                manifest[-1].update(algorithmic_bytes=item.algorithmic_bytes, workload=item.workload)
        finally:
            rt.finalize()
    os.makedirs(os.path.dirname(args.manifest), exist_ok=True)
    with open(args.manifest, "w") as fh:
        json.dump(manifest, fh, indent=1)
    print("profile_workloads: %d workloads, manifest %s" % (len(manifest), args.manifest))


if __name__ == "__main__":
    main()
