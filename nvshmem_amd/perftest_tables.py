"""Runs the command-line driver nvshmem_amd/bin/nvshmem_perftest over the size sweeps of the put/get
configuration and over the in-kernel latency tests, and writes what it printed as the two text tables
kept under profiles/:

    python3 nvshmem_amd/perftest_tables.py --what put_get  --out profiles/put_get_sweep.txt
    python3 nvshmem_amd/perftest_tables.py --what latency  --out profiles/in_kernel_latency.txt
    python3 nvshmem_amd/perftest_tables.py --what collectives --out profiles/collective_size_sweep.txt

put_get  putmem_block / getmem_block between 8 logical PEs (PE p and (p + 1) % 8), 8 B to 256 MiB per PE
         in powers of two, from 1 / 4 / 16 blocks of 1024 threads per PE (block b moves the b-th
         contiguous slice).  The driver reports the payload of one PE per second, as the reference's
         perftest/device/pt-to-pt/shmem_put_bw.cu:268 does; the table adds the time of one exchange, the
         payload of all 8 PEs, the bytes read and written (twice the payload) and that figure's share of
         the 8 TB/s HBM peak.
latency  barrier_all / sync_all, put and get of one thread group with quiet, put_signal ping-pong, and
         the five collectives at 8 B to 4 KiB per PE, all called in a loop inside one kernel (the
         reference's perftest/device/coll/*_latency.cu and perftest/device/pt-to-pt/*latency.cu shapes).

collectives  the host-launched (on-stream) reduce, fcollect, broadcast, alltoall and reducescatter from 256 KiB
         to 128 MiB per PE, as the library chooses its kernels and with each of the two forms forced through
         the environment (NVSHMEM_AMD_LDS_REDUCE_BYTES, NVSHMEM_AMD_CHUNKED_COPY_BYTES): the evidence for the
         sizes at which the library switches.  Times are host wall time per call over back-to-back calls,
         so the smallest sizes show the launch rate, and sources up to 256 MiB in all stay in the Infinity
         Cache from one call to the next.

Every table lists the driver commands that produced it; the sweep follows the reference's
perftest/common/utils.cu:859-873 (sizes in powers of two between --min and --max).
"""
import argparse
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "nvshmem_amd", "bin", "nvshmem_perftest")
HBM_PEAK_GBS = 8000.0
NPES = 8


def run_driver(args, env=None):
    """-> (command line as text, stdout).  Fails loudly: a table must not be built from a failed run."""
    cmd = [DRIVER] + args
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                          env=dict(os.environ, **env) if env else None)
    shown = " ".join(["%s=%s" % kv for kv in sorted((env or {}).items())] +
                     ["nvshmem_amd/bin/nvshmem_perftest " + " ".join(args)])
    if proc.returncode != 0:
        raise SystemExit("%s failed (%d):\n%s" % (shown, proc.returncode, proc.stderr))
    return shown, proc.stdout


def rows_of(text):
    """Rows 'size scope value' of a driver table -> [(size, value)]."""
    out = []
    for line in text.splitlines():
        m = re.match(r"^(\d+)\s+\S+\s+([0-9.eE+-]+)\s*$", line)
        if m:
            out.append((int(m.group(1)), float(m.group(2))))
    return out


def put_get(iters):
    lines, commands = [], []
    for test, api in (("put_bw", "nvshmemx_putmem_block"), ("get_bw", "nvshmemx_getmem_block")):
        for blocks in (1, 4, 16):
            shown, text = run_driver([test, "--npes", str(NPES), "--min", "8", "--max", "256m", "--blocks", str(blocks),
                                      "--threads", "1024", "--scope", "block", "--iters", str(iters)])
            commands.append(shown)
            lines += ["", "%s, %d logical PEs, %d block%s x 1024 threads per PE" % (api, NPES, blocks, "" if blocks == 1 else "s"),
                      "%12s %12s %16s %18s %20s %10s" % ("bytes per PE", "us", "GB/s per PE", "payload GB/s (all)",
                                                         "read + write GB/s", "of peak")]
            for size, gbs in rows_of(text):
                us = size / gbs / 1e3 if gbs > 0 else float("nan")
                lines.append("%12d %12.2f %16.2f %18.1f %20.1f %10.4f" % (size, us, gbs, NPES * gbs, 2 * NPES * gbs,
                                                                         2 * NPES * gbs / HBM_PEAK_GBS))
    head = ["put / get size sweep (configuration: message sizes 8 B to 256 MiB in powers of two, 1 / 4 / 16 concurrent",
            "blocks per PE), one MI355X, all PEs carried by one launch; times include the kernel launch (a few us),",
            "which is what bounds the rows up to about 256 KiB.", "",
            "Commands (repository root, after python3 -m nvshmem_amd.build):",
            "  python3 nvshmem_amd/perftest_tables.py --what put_get --out profiles/put_get_sweep.txt", "which runs"]
    return head + ["  " + c for c in commands] + lines


def latency(iters):
    lines, commands = [], []
    jobs = [["barrier_latency", "--scope", "block"], ["barrier_latency", "--scope", "warp"], ["barrier_latency", "--scope", "thread"],
            ["sync_latency", "--scope", "block"],
            ["pt2pt_latency", "--min", "8", "--max", "4k"],
            ["coll_latency", "--min", "8", "--max", "4k", "--scope", "block"],
            ["coll_latency", "--min", "8", "--max", "4k", "--scope", "warp"]]
    for job in jobs:
        shown, text = run_driver([job[0], "--npes", str(NPES), "--iters", str(iters)] + job[1:])
        commands.append(shown)
        lines += ["", "$ " + shown] + [l.rstrip() for l in text.splitlines()]
    head = ["In-kernel latencies, 8 logical PEs on one MI355X: the call is repeated inside one kernel and the time of",
            "a launch with one call is subtracted, so a figure is the cost of one more call.  Sizes are bytes per PE.", "",
            "Commands (repository root, after python3 -m nvshmem_amd.build):",
            "  python3 nvshmem_amd/perftest_tables.py --what latency --out profiles/in_kernel_latency.txt", "which runs"]
    return head + ["  " + c for c in commands] + lines


def bandwidth_rows(text):
    """The 'algorithmic BW' table of a host collective run -> [(bytes per PE, GB/s)]."""
    out, inside = [], False
    for line in text.splitlines():
        if line.startswith("size(B)"):
            inside = "BW" in line
            continue
        m = re.match(r"^(\d+)\s+\S+\s+([0-9.eE+-]+)\s*$", line)
        if m and inside:
            out.append((int(m.group(1)), float(m.group(2))))
    return out


def collectives(iters):
    never = str(1 << 40)
    jobs = [("reduce (fp32 sum)", "reduce", npes, "128m" if npes <= 8 else "32m" if npes <= 16 else "16m",
             (("library's choice", {}), ("LDS-staged kernel at every size", {"NVSHMEM_AMD_LDS_REDUCE_BYTES": "0"}),
              ("gather kernel at every size", {"NVSHMEM_AMD_LDS_REDUCE_BYTES": never,
                                               "NVSHMEM_AMD_TWO_STEP_REDUCE_MEMBERS": "0"})))
            for npes in (4, 8, 16, 32, 64)]
    jobs += [("fcollect", "fcollect", npes, "32m" if npes <= 8 else "16m",
              (("library's choice", {}), ("chunked form at every size", {"NVSHMEM_AMD_CHUNKED_COPY_BYTES": "0"}),
               ("plain form at every size", {"NVSHMEM_AMD_CHUNKED_COPY_BYTES": never}))) for npes in (4, 8, 16)]
    jobs += [("broadcast", "broadcast", 8, "128m",
              (("library's choice", {}), ("chunked form at every size", {"NVSHMEM_AMD_CHUNKED_COPY_BYTES": "0"}),
               ("plain form at every size", {"NVSHMEM_AMD_CHUNKED_COPY_BYTES": never}))),
             ("alltoall (bytes per destination)", "alltoall", 8, "16m", (("library's choice", {}),)),
             ("reducescatter (bytes per block)", "reducescatter", 8, "16m", (("library's choice", {}),))]
    lines, commands = [], []
    for title, test, npes, top, forms in jobs:
        table, sizes = [], None
        for label, env in forms:
            shown, text = run_driver([test, "--npes", str(npes), "--min", "256k", "--max", top, "--iters", str(iters)], env)
            commands.append(shown)
            rows = bandwidth_rows(text)
            sizes = sizes or [s for s, _ in rows]
            table.append((label, dict(rows)))
        lines += ["", "%s, %d logical PEs: algorithmic GB/s by bytes per PE" % (title, npes),
                  "%-34s" % "form" + "".join("%8s" % ("%dK" % (s >> 10) if s < 1 << 20 else "%dM" % (s >> 20)) for s in sizes)]
        for label, rows in table:
            lines.append("%-34s" % label + "".join("%8.0f" % rows.get(s, float("nan")) for s in sizes))
    head = ["Host-launched collectives by size on one MI355X: what the library's kernel choice gives, and what each of",
            "the two forms it chooses between gives when forced through the environment.  Algorithmic bytes as in",
            "bench.py; host wall time over back-to-back calls (a call costs at least a launch, ~3 us; sources up to",
            "256 MiB in all stay in the Infinity Cache between calls).", "",
            "Commands (repository root, after python3 -m nvshmem_amd.build):",
            "  python3 nvshmem_amd/perftest_tables.py --what collectives --out profiles/collective_size_sweep.txt", "which runs"]
    return head + ["  " + c for c in commands] + lines


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--what", required=True, choices=("put_get", "latency", "collectives"))
    ap.add_argument("--out", required=True)
    ap.add_argument("--iters", type=int, default=0)
    args = ap.parse_args()
    if not os.path.exists(DRIVER):
        raise SystemExit("%s is not built (python3 -m nvshmem_amd.build)" % DRIVER)
    lines = (put_get(args.iters or 20) if args.what == "put_get" else
             latency(args.iters or 200) if args.what == "latency" else collectives(args.iters or 40))
    os.makedirs(os.path.dirname(os.path.abspath(args.out)), exist_ok=True)
    with open(args.out, "w") as fh:
        fh.write("\n".join(lines) + "\n")
    print("perftest_tables: wrote %s (%d lines)" % (args.out, len(lines)))


if __name__ == "__main__":
    sys.exit(main())
