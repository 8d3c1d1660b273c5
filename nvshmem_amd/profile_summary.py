"""Turns rocprofv3 result databases (rocpd / sqlite) into the short text summary kept under
profiles/.

    python3 nvshmem_amd/profile_summary.py --stats <dir> [--fetch <dir>] [--write <dir>]

Each <dir> is a rocprofv3 `-d` output directory.  Per kernel: calls and average duration from the
kernel trace; average FETCH_SIZE / WRITE_SIZE (KiB per dispatch) from the counter runs, and the
same scaled by what the counter reads for the plain copy calibration kernel, whose traffic is known
(1 GiB read, 1 GiB written).
"""
import argparse
import glob
import os
import sqlite3

CALIBRATION = "plain_copy_kernel"
CALIBRATION_KIB = float(1 << 20)   # 1 GiB in KiB, read and written


def _db(directory):
    hits = sorted(glob.glob(os.path.join(directory, "**", "*_results.db"), recursive=True),
                  key=os.path.getmtime)
    if not hits:
        raise SystemExit("no *_results.db under %s" % directory)
    return sqlite3.connect(hits[-1])


def _short(name):
    name = name.replace("nvshmem_amd::(anonymous namespace)::", "").replace("(anonymous namespace)::", "")
    name = name.replace("void ", "")
    return name.split("(")[0]


def kernel_stats(directory):
    cur = _db(directory).cursor()
    rows = cur.execute("select name, count(*), avg(duration), min(duration), max(duration) "
                       "from kernels group by name order by sum(duration) desc").fetchall()
    return [(_short(n), c, a / 1e3, lo / 1e3, hi / 1e3) for n, c, a, lo, hi in rows]


def counter_avg(directory, counter):
    cur = _db(directory).cursor()
    rows = cur.execute("select kernel_name, avg(value), count(*) from counters_collection "
                       "where counter_name = ? group by kernel_name", (counter,)).fetchall()
    return {_short(n): (v, c) for n, v, c in rows}


# workloads of nvshmem_amd/profile_workloads.py:
# leading part of the kernel name as the trace prints it -> (file name, description, algorithmic bytes)
WORKLOADS = {
    "ring_rma_kernel<2, false>": (
        "ring_rma_kernel_put_block_8pe_256MiB.txt",
        "put_block: nvshmemx_putmem_block ring, 8 logical PEs x 256 MiB, 262144 blocks x 64 threads per PE (1 KiB per block).\n"
        "Algorithmic bytes per launch: 8 x 256 MiB read + 8 x 256 MiB written = 4 GiB.", 4 << 30),
    "reduce_vector_kernel<float, 5, 8, true,": (
        "reduce_vector_kernel_float_sum_8pe_64Mi.txt",
        "sum_reduce: nvshmemx_float_sum_reduce_on_stream, 8 logical PEs x 2^26 fp32.\n"
        "Algorithmic bytes per launch: 8 sources read once + 8 destinations written once = 4 GiB.", 4 << 30),
    "segment_copy_kernel<1, 1, false>": (
        "segment_copy_kernel_alltoall_16pe_4Mi_fp32.txt",
        "alltoall: nvshmemx_float_alltoall_on_stream, 16 logical PEs x 2^22 fp32 (block 2^18 elements).\n"
        "Algorithmic bytes per launch: 256 MiB read + 256 MiB written = 512 MiB.  The 256 MiB source fits the\n"
        "Infinity Cache and the profiled loop re-sends it; FETCH_SIZE counts between L2 and the fabric and\n"
        "cannot tell a cache hit from an HBM read, but a rate above the HBM peak shows that part of the\n"
        "reads are served by the cache.", 512 << 20),
    "segment_copy_kernel<0, 1, false>": (
        "segment_copy_kernel_fcollect_16pe_4Mi_fp32.txt",
        "fcollect: nvshmemx_float_fcollect_on_stream, 16 logical PEs x 2^22 fp32.\n"
        "Algorithmic bytes per launch: 256 MiB read + 16 x 256 MiB written = 4.25 GiB.", (17 * 256) << 20),
    "reducescatter_gather_kernel<float, 5, 8, true>": (
        "reducescatter_gather_kernel_float_sum_8pe_8Mi.txt",
        "reducescatter: nvshmemx_float_sum_reducescatter_on_stream, 8 logical PEs, source 8 x 2^23 fp32\n"
        "(256 MiB) per PE, result 2^23 fp32 (32 MiB) per PE.\n"
        "Algorithmic bytes per launch: 8 sources of 256 MiB read once + 8 results of 32 MiB written = 2.25 GiB.",
        (9 * 256) << 20),
    "segment_copy_kernel<2, 1, false>": (
        "segment_copy_kernel_broadcast_8pe_256MiB.txt",
        "broadcast: nvshmemx_broadcastmem_on_stream, 8 logical PEs, 256 MiB from PE 3.\n"
        "Algorithmic bytes per launch: 256 MiB read + 8 x 256 MiB written = 2.25 GiB.", (9 * 256) << 20),
    "moe_dispatch_direct_kernel<1>": (
        "moe_dispatch_direct_kernel_8pe_8192tok_top8.txt",
        "MoE dispatch (config 5): 8 logical PEs x 8192 tokens x 7168 bf16, top-8 of 256 experts, Zipf(1.1);\n"
        "1 KiB work items, at most four copies per wavefront: two neighbouring blocks share a piece.  They run on\n"
        "different XCDs, so both fetch it through the fabric (FETCH_SIZE counts it twice); the second fetch is\n"
        "served by the Infinity Cache, not by HBM.  The signalling kernel that follows\n"
        "(moe_dispatch_signal_kernel) is not part of this figure.\n"
        "Algorithmic bytes per launch: every row read once (896 MiB) + written 8 times (7 GiB) = 7.875 GiB.",
        (896 + 7168) << 20),
    "moe_combine_kernel<true, 2048>": (
        "moe_combine_kernel_8pe_8192tok_top8.txt",
        "MoE combine (config 5): every one of the 8 x 65536 row copies fetched back with nvshmemx_getmem_nbi_warp,\n"
        "2 KiB per single-wavefront block.\n"
        "Algorithmic bytes per launch: 7 GiB read + 7 GiB written = 14 GiB.", 14 << 30),
    "plain_copy_kernel": (
        "plain_copy_kernel_calibration_1GiB.txt",
        "Counter calibration: plain one-vector-per-thread copy, 1 GiB read + 1 GiB written.", 2 << 30),
}

COMMANDS = """Commands (from the repository root on the GPU box; every file they run is committed):
  cd /tmp && export TMPDIR=/tmp OUT=<a scratch directory>
  rocprofv3 --kernel-trace --stats -d $OUT/prof_stats -- python3 $REPO/nvshmem_amd/profile_workloads.py
  rocprofv3 --pmc FETCH_SIZE -d $OUT/prof_fetch -- python3 $REPO/nvshmem_amd/profile_workloads.py --iters 5
  rocprofv3 --pmc WRITE_SIZE -d $OUT/prof_write -- python3 $REPO/nvshmem_amd/profile_workloads.py --iters 5
  python3 nvshmem_amd/profile_summary.py --stats $OUT/prof_stats --fetch $OUT/prof_fetch \\
          --write $OUT/prof_write --profiles-dir profiles
Hardware: one MI355X (gfx950), ROCm 7.2.  Durations are per dispatch from the kernel trace."""


def write_profiles(directory, stats, fetch, write, fscale, wscale):
    os.makedirs(directory, exist_ok=True)
    def find(table, prefix):
        hits = [k for k in table if k.startswith(prefix)]
        return hits[0] if len(hits) == 1 else None

    by_name = {s[0]: s for s in stats}
    for prefix, (fname, desc, alg) in WORKLOADS.items():
        kernel = find(by_name, prefix)
        if kernel is None:
            continue
        name, calls, avg, lo, hi = by_name[kernel]
        lines = [desc, "", COMMANDS, "",
                 "%-46s %6s %12s %12s %12s" % ("kernel", "calls", "avg us", "min us", "max us"),
                 "%-46s %6d %12.2f %12.2f %12.2f" % (name[:46], calls, avg, lo, hi), "",
                 "full kernel name: " + name, ""]
        if fscale and wscale and kernel in fetch and kernel in write:
            f, w = fetch[kernel][0], write[kernel][0]
            lines += ["counters (KiB per dispatch): FETCH_SIZE %.1f  WRITE_SIZE %.1f" % (f, w),
                      "scale factors from plain_copy_kernel (1 GiB read + 1 GiB written): "
                      "FETCH_SIZE x%.4f, WRITE_SIZE x%.4f" % (fscale, wscale),
                      "HBM traffic per dispatch (scaled): read %.1f MiB + written %.1f MiB = %.1f MiB; "
                      "algorithmic bytes %.1f MiB" % (f * fscale / 1024, w * wscale / 1024,
                                                      (f * fscale + w * wscale) / 1024, alg / 2**20), ""]
        lines.append("achieved = algorithmic bytes / average duration = %.0f GB/s = %.1f %% of the "
                     "8000 GB/s HBM peak" % (alg / avg / 1e3, alg / avg / 1e3 / 80.0))
        with open(os.path.join(directory, fname), "w") as fh:
            fh.write("\n".join(lines) + "\n")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--stats", required=True)
    ap.add_argument("--fetch")
    ap.add_argument("--write")
    ap.add_argument("--profiles-dir", help="also write one summary file per workload there")
    args = ap.parse_args()
    stats = kernel_stats(args.stats)
    fetch = counter_avg(args.fetch, "FETCH_SIZE") if args.fetch else {}
    write = counter_avg(args.write, "WRITE_SIZE") if args.write else {}
    fscale = CALIBRATION_KIB / fetch[CALIBRATION][0] if CALIBRATION in fetch else None
    wscale = CALIBRATION_KIB / write[CALIBRATION][0] if CALIBRATION in write else None
    print("%-46s %6s %12s %12s %12s" % ("kernel", "calls", "avg us", "min us", "max us"))
    for name, calls, avg, lo, hi in stats:
        print("%-46s %6d %12.2f %12.2f %12.2f" % (name[:46], calls, avg, lo, hi))
    if fetch or write:
        print()
        print("counter scale factors from %s (known 1 GiB read + 1 GiB written): FETCH_SIZE x%s, "
              "WRITE_SIZE x%s" % (CALIBRATION, "%.4f" % fscale if fscale else "n/a",
                                  "%.4f" % wscale if wscale else "n/a"))
        print("%-46s %14s %14s %14s %14s" % ("kernel", "FETCH KiB", "WRITE KiB", "read MiB (scaled)",
                                             "write MiB (scaled)"))
        for name in sorted(set(fetch) | set(write)):
            f = fetch.get(name, (float("nan"), 0))[0]
            w = write.get(name, (float("nan"), 0))[0]
            fs = f * fscale / 1024 if fscale else float("nan")
            ws = w * wscale / 1024 if wscale else float("nan")
            print("%-46s %14.1f %14.1f %14.1f %14.1f" % (name[:46], f, w, fs, ws))
    if args.profiles_dir:
        write_profiles(args.profiles_dir, stats, fetch, write, fscale, wscale)


if __name__ == "__main__":
    main()
