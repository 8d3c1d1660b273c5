#!/usr/bin/env python3
"""Benchmark of the NVSHMEM data-movement hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only name,name]

Prints ONE JSON line.  The headline workload is put_block on the put/get sweep's own launch shape at
its largest size: every one of 8 logical PEs moves 256 MiB to its right neighbour with
nvshmemx_putmem_block from 16 blocks of 1024 threads, block b moving the b-th contiguous slice; a
"step" is one such exchange (one kernel launch carrying all PEs).  `value` is algorithmic bytes
(payload read once + written once, all PEs) per second, inputs already resident in HBM.  Every other
configuration of the sweep - put and get at 64 and 256 MiB from 1 / 4 / 16 blocks, the launch shape
that fills the GPU, the reductions, fcollect / alltoall, reducescatter, broadcast and the MoE token
shuffle - is measured the same way and reported under "workloads", each verified against the CPU
oracle and each with the oracle's own rate on this host (one thread, and all threads OpenMP gives).
"""
import argparse
import glob
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0   # MI355X published HBM3E peak
METRIC = "achieved GB/s and % of HBM peak: put_block, sum_reduce, alltoall (1 GPU)"


def measured_traffic(name, fingerprint):
    """HBM bytes per launch of the workload's dominant kernel, from the rocprofv3 FETCH_SIZE / WRITE_SIZE
    summary committed under profiles/.  None when there is no summary, or when the summary was measured
    on kernel sources other than the ones in this tree (it records their fingerprint)."""
    for path in glob.glob(os.path.join(ROOT, "profiles", "*__%s.txt" % name)):
        with open(path) as fh:
            text = fh.read()
        m = re.search(r"^measured_traffic_bytes: (\d+) read \+ (\d+) written", text, re.M)
        f = re.search(r"^kernel_sources_fingerprint: (\w+)", text, re.M)
        if m and f and f.group(1) == fingerprint:
            return int(m.group(1)) + int(m.group(2))
    return None


def time_steps(fn, steps, warmup, hip):
    """(wall ms per step, event ms per step): K launches bracketed by device synchronisation."""
    for _ in range(warmup):
        fn()
    hip.synchronize()
    e0, e1 = hip.Event(), hip.Event()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    hip.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    ev = e0.elapsed_ms(e1) / steps
    e0.destroy(); e1.destroy()
    return wall, ev


def cpu_time(fn, budget_s, max_passes=20):
    best, spent, passes = None, 0.0, 0
    while passes < max_passes and (spent < budget_s or passes == 0):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
        spent += dt
        passes += 1
    return best, passes


class Checker:
    """Verification against the oracle and the oracle's own rate, per kind of workload."""

    def __init__(self, O, np, cpu_seconds):
        self.O, self.np, self.budget = O, np, cpu_seconds
        self.cores = O.lib().oracle_get_threads()      # what OpenMP gives this process on this host

    def baseline(self, fn, bytes_moved, sample):
        """Two rows: one thread, and all threads."""
        O = self.O
        O.lib().oracle_set_threads(1)
        one, _ = cpu_time(fn, self.budget / 2)
        O.lib().oracle_set_threads(self.cores)
        best, passes = cpu_time(fn, self.budget / 2)
        return {"value": round(bytes_moved / best / 1e9, 2), "unit": "GB/s", "cores": self.cores, "kind": "port",
                "sample": "%s, best of %d passes" % (sample, passes),
                "single_thread": round(bytes_moved / one / 1e9, 2)}

    # -- put / get ---------------------------------------------------------------------------
    def rma_prepare(self, g, item):
        g.rt.fill(g.dst, 0, item.config["bytes_per_pe"])

    def rma_verify(self, g, item):
        np, size, npes = self.np, item.config["bytes_per_pe"], g.npes
        shift = 1 if item.config["is_get"] else -1
        return all(bool(np.array_equal(g.rt.download(g.dst, pe, (size,), np.uint8), g.data[(pe + shift) % npes][:size]))
                   for pe in range(npes))

    def rma_baseline(self, g, item):
        np, sample = self.np, 32 << 20
        if not hasattr(g, "_host"):
            g._host = (np.ascontiguousarray(g.data[:, :sample]), np.zeros((g.npes, sample), np.uint8))
        src, dst = g._host
        fn = (lambda: self.O.ring_get(src)) if item.config["is_get"] else (lambda: self.O.ring_put(src, dst))
        return self.baseline(fn, 2 * g.npes * sample,
                             "oracle_ring_%s (memcpy), 8 PEs x 32 MiB" % ("get" if item.config["is_get"] else "put"))

    # -- allreduce ---------------------------------------------------------------------------
    def reduce_prepare(self, g, item):
        item.prepare()

    def reduce_verify(self, g, item):
        np, O = self.np, self.O
        data = g.data["array"]
        n, es = g.n, item.elem_bytes
        ok = True
        for lo, cnt in ((0, min(n, 1 << 22)), (max(0, n - (1 << 16)), min(n, 1 << 16))):
            want = O.reduce(item.oracle_dtype, item.op, data[:, lo:lo + cnt])
            for pe in sorted({0, min(5, g.npes - 1), g.npes - 1}):
                got = g.rt.download(g.dst, pe, (cnt,), want.dtype, lo * es)
                ok = ok and bool(np.array_equal(got.view(np.uint8), want.view(np.uint8)))
        return ok

    def reduce_baseline(self, g, item):
        np = self.np
        cs = min(g.n, 1 << 22)
        host = np.ascontiguousarray(g.data["array"][:, :cs])
        # the oracle produces one PE's result, so its figure counts what it moves: npes reads + 1 write
        return self.baseline(lambda: self.O.reduce(item.oracle_dtype, item.op, host), (g.npes + 1) * cs * item.elem_bytes,
                             "oracle_reduce %s %s, %d PEs x %d elements (%d reads + 1 write per element)"
                             % (item.oracle_dtype, item.op, g.npes, cs, g.npes))

    # -- fcollect / alltoall -------------------------------------------------------------------
    def collect_prepare(self, g, item):
        pass

    def collect_verify(self, g, item):
        np, npes = self.np, g.npes
        nbytes = g.n * g.es
        if item.what == "alltoall":
            want = self.O.alltoall(g.data)
            return all(bool(np.array_equal(g.rt.download(g.a2a_dst, pe, (nbytes,), np.uint8), want[pe]))
                       for pe in range(npes))
        want = g.data.reshape(-1)                      # every PE: the sources in PE order
        return all(bool(np.array_equal(g.rt.download(g.fc_dst, pe, (npes * nbytes,), np.uint8), want))
                   for pe in (0, 9, 15))

    def collect_baseline(self, g, item):
        np, npes = self.np, g.npes
        seg = (1 << 20) if item.what == "alltoall" else (1 << 18)     # bytes per (source, destination) / per source
        if item.what == "alltoall":
            host = np.ascontiguousarray(g.data[:, :npes * seg])
            return self.baseline(lambda: self.O.alltoall(host), 2 * npes * npes * seg,
                                 "oracle_alltoall, 16 PEs x 16 MiB")
        host = np.ascontiguousarray(g.data[:, :seg * 16])
        return self.baseline(lambda: self.O.fcollect(host), (npes + 1) * npes * seg * 16,
                             "oracle_fcollect, 16 PEs x 4 MiB")

    # -- reducescatter / broadcast ---------------------------------------------------------------
    def reducescatter_prepare(self, g, item):
        pass

    def reducescatter_verify(self, g, item):
        np, npes, n, sample = self.np, g.npes, g.n, 1 << 20
        want = self.O.reducescatter("f32", "sum", np.ascontiguousarray(
            g.data.reshape(npes, npes, n)[:, :, :sample].reshape(npes, npes * sample)))
        return all(bool(np.array_equal(g.rt.download(g.dst, pe, (sample,), np.float32).view(np.uint32),
                                       want[pe].view(np.uint32))) for pe in (0, 5))

    def reducescatter_baseline(self, g, item):
        np, npes, cs = self.np, g.npes, 1 << 19
        host = np.ascontiguousarray(g.data[:, :npes * cs])
        return self.baseline(lambda: self.O.reducescatter("f32", "sum", host), (npes + 1) * npes * cs * 4,
                             "oracle_reducescatter f32 sum, 8 PEs x 8 x 2^19 elements")

    def broadcast_prepare(self, g, item):
        pass

    def broadcast_verify(self, g, item):
        np = self.np
        return all(bool(np.array_equal(g.rt.download(g.dst, pe, (g.nbytes,), np.uint8), g.row)) for pe in (0, 3, 7))

    def broadcast_baseline(self, g, item):
        np, sample = self.np, 32 << 20
        host = np.ascontiguousarray(np.broadcast_to(g.row[:sample], (g.npes, sample)))
        return self.baseline(lambda: self.O.broadcast(host, g.root), (g.npes + 1) * sample,
                             "oracle_broadcast (memcpy per PE), 8 PEs x 32 MiB")

    # -- MoE -----------------------------------------------------------------------------------
    def moe_prepare(self, g, item):
        item.prepare()
        if item.what != "combine":
            g.rt.fill(g.recv, 0, g.cap * g.row)

    def moe_verify(self, g, item):
        np, rt = self.np, g.rt
        npes, K, row, rows = g.npes, g.K, g.row, g.rows
        ok = all(rt.read_timeout(pe)[0] == 0 for pe in range(npes))
        if item.what in ("put_signal", "put_signal_head"):
            sig = rt.download_all(g.sig, (npes * g.SIG_STRIDE,), np.uint64)[:, ::g.SIG_STRIDE]
            ok = ok and bool(np.array_equal(sig, g.expected if item.what == "put_signal" else g.expected_head))
        if item.what == "put_signal_head":
            rows = g.FULL_ORDER_TOKENS * K       # only the first tokens were sent
        elif item.what == "plain_store":
            ok = ok and bool(np.array_equal(rt.download_all(g.sig, (npes,), np.uint64), g.expected))
        rng = np.random.default_rng(0)
        for src_pe in range(npes):
            for r in rng.integers(0, rows, 128):
                got = rt.download(g.recv, int(g.dest_pe[src_pe, r]), (row,), np.uint8, int(g.dest_row[src_pe, r]) * row)
                ok = ok and bool(np.array_equal(got, g.payload[src_pe, r // K]))
                if item.what == "combine":
                    back = rt.download(g.out, src_pe, (row,), np.uint8, int(r) * row)
                    ok = ok and bool(np.array_equal(back, got))
        return ok

    def moe_baseline(self, g, item):
        np, O = self.np, self.O
        npes, K, E, row, Ts = g.npes, g.K, g.E, g.row, 512
        if not hasattr(g, "_small"):
            exs = O.moe_routing(npes, Ts, K, E, 1.1, 8)
            _, _, s_pe, s_row, s_recv = O.moe_plan(exs, npes, Ts, K, E)
            small = np.ascontiguousarray(g.payload[:, :Ts])
            g._small = (small, s_pe, s_row, s_recv, O.moe_dispatch(small, s_pe, s_row, s_recv, Ts, K))
        small, s_pe, s_row, s_recv, held = g._small
        moved = npes * Ts * K * row
        if item.what == "combine":
            return self.baseline(lambda: O.moe_combine(held, s_pe, s_row, Ts, K, row), 2 * moved,
                                 "oracle_moe_combine, 512 tokens per PE")
        return self.baseline(lambda: O.moe_dispatch(small, s_pe, s_row, s_recv, Ts, K), moved + moved // K,
                             "oracle_moe_dispatch, 512 tokens per PE")


def oracle_moe_plan(O, np, npes, T, K, E):
    ex = O.moe_routing(npes, T, K, E, 1.1, 8)
    counts, _, dest_pe, dest_row, recv_rows = O.moe_plan(ex, npes, T, K, E)
    epp = E // npes
    expected = np.stack([[counts[s, d * epp:(d + 1) * epp].sum() for s in range(npes)]
                         for d in range(npes)]).astype(np.uint64)
    return dest_pe, dest_row, expected, recv_rows


def summarise(item, wall, ev, ok, cpu, fingerprint):
    gbs = item.algorithmic_bytes / wall / 1e6
    kernel_gbs = item.algorithmic_bytes / ev / 1e6
    cfg = dict(item.config, workload=item.workload)
    if "bytes_per_pe" in item.config:
        cfg["payload_only_GBs"] = round(item.config["npes"] * item.config["bytes_per_pe"] / ev / 1e6, 1)
    cached = bool(getattr(item, "cache_resident", False))      # then the rate is no HBM figure: no fraction
    return {
        "GBs": round(gbs, 1), "frac_of_hbm_peak": None if cached else round(gbs / HBM_PEAK_GBS, 4),
        "ms_per_step": round(wall, 5), "kernel_ms": round(ev, 5), "kernel_GBs": round(kernel_gbs, 1),
        "kernel_frac_of_hbm_peak": None if cached else round(kernel_gbs / HBM_PEAK_GBS, 4),
        "cache_resident": cached,
        "algorithmic_bytes": item.algorithmic_bytes, "traffic": measured_traffic(item.name, fingerprint),
        "dtype": item.dtype, "verified": ok, "config": cfg, "kernel": item.kernel, "cpu_baseline": cpu,
    }


MAX_LINE_BYTES = 4096    # the result line is read back from a bounded tail of stdout


def result_line(results, headline, warmup):
    """The ONE result line, from the per-workload records of summarise(): the headline workload's figures
    in full, every other workload as [kernel GB/s, fraction of the HBM peak or None when the working set
    stays in the Infinity Cache, verified].  Kept well under MAX_LINE_BYTES; the full records are printed
    on earlier lines."""
    head = results[headline]
    cpu = dict(head["cpu_baseline"])
    config = {k: v for k, v in head["config"].items() if k != "note"}
    line = {
        "metric": METRIC,
        "value": head["GBs"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": head["steps"],
        "warmup": warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic",
        "config": config,
        "roofline": {"bound": "hbm", "achieved": head["kernel_GBs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(head["kernel_GBs"] / HBM_PEAK_GBS, 4), "traffic": head["traffic"],
                     "kernel": head["kernel"]},
        "cpu_baseline": cpu,
        "verified": all(r["verified"] for r in results.values()),
        "workloads_format": "name: [kernel GB/s, fraction of HBM peak (null: cache resident), verified]",
        "workloads": {name: [r["kernel_GBs"], r["kernel_frac_of_hbm_peak"], r["verified"]]
                      for name, r in results.items()},
    }
    if len(json.dumps(line, separators=(",", ":"))) >= MAX_LINE_BYTES:
        raise RuntimeError("bench.py: the result line outgrew %d bytes" % MAX_LINE_BYTES)
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-seconds", type=float, default=1.5, help="CPU oracle timing budget per workload")
    ap.add_argument("--only", default="", help="comma-separated workload names (the headline always runs)")
    ap.add_argument("--trace-manifest", default="",
                    help="for runs under rocprofv3: bracket every workload's launches with the empty "
                         "profile_marker_kernel and write the order of the workloads to this file, so that "
                         "nvshmem_amd/profile_summary.py can cut the kernel trace into workloads")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs all logical PEs on ONE GPU; --gpus %d is not supported "
              "(no inter-GPU path exists)" % args.gpus, file=sys.stderr)
        return 2

    import numpy as np
    import nvshmem_amd as N          # raises if the HIP libraries are not built
    from nvshmem_amd import hip, workloads
    from nvshmem_amd.fingerprint import kernel_source_fingerprint
    import oracle_lib as O           # the checker / CPU baseline only
    fingerprint = kernel_source_fingerprint()

    if hip.device_count() < 1:
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3

    only = set(x for x in args.only.split(",") if x)
    if only:
        only.add(workloads.HEADLINE)
    check = Checker(O, np, args.cpu_seconds)
    results, manifest = {}, []
    groups = workloads.all_groups(oracle_moe_plan(O, np, 8, 8192, 8, 256))
    for g in groups:
        if only and not any(n in only for n in g.names()):
            continue
        rt = N.Runtime(npes=g.npes, symmetric_size=g.heap_bytes)
        try:
            for item in g.setup(rt, O.fill_all):
                if only and item.name not in only:
                    continue
                getattr(check, g.kind + "_prepare")(g, item)
                steps, warmup = max(1, args.steps // item.scale), max(1, args.warmup // item.scale)
                if args.trace_manifest:
                    rt.perftest().nvshmem_perftest_profile_marker(None)
                wall, ev = time_steps(item.step, steps, warmup, hip)
                if args.trace_manifest:
                    rt.perftest().nvshmem_perftest_profile_marker(None)
                    hip.synchronize()
                    manifest.append({"name": item.name, "launches": steps + warmup, "workload": item.workload,
                                     "algorithmic_bytes": item.algorithmic_bytes})
                ok = getattr(check, g.kind + "_verify")(g, item)
                cpu = getattr(check, g.kind + "_baseline")(g, item)
                results[item.name] = summarise(item, wall, ev, ok, cpu, fingerprint)
                results[item.name]["steps"] = steps
        finally:
            rt.finalize()

    if args.trace_manifest:
        with open(args.trace_manifest, "w") as fh:
            json.dump(manifest, fh, indent=1)
    for name, rec in results.items():          # the full records, one line per workload, before the result line
        print(json.dumps({"workload_record": name, **rec}))
    line = result_line(results, workloads.HEADLINE, args.warmup)
    print(json.dumps(line, separators=(",", ":")))
    sys.stdout.flush()
    return 0 if line["verified"] else 1


if __name__ == "__main__":
    sys.exit(main())
