"""Turns rocprofv3 result databases (rocpd / sqlite) of nvshmem_amd/profile_workloads.py runs into the
short text summaries kept under profiles/, one per workload.

    python3 nvshmem_amd/profile_summary.py --manifest <json> --stats <dir> [--pmc <dir> ...]
                                           [--profiles-dir profiles] [--only name,name]

Each <dir> is a rocprofv3 `-d` output directory: --stats from a `--kernel-trace --stats` run, every
--pmc from one `--pmc <counters>` run.  profile_workloads.py brackets each workload with two launches
of profile_marker_kernel and records the order in the manifest, so dispatches are assigned to workloads
by counting markers.  Per workload and kernel: calls and average / min / max duration; per counter the
average per dispatch; FETCH_SIZE / WRITE_SIZE (KiB per dispatch) also scaled by what the same counter
reads for the calibration workload, a plain copy kernel of known traffic (1 GiB read, 1 GiB written).
"""
import argparse
import glob
import json
import os
import re
import sqlite3
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from nvshmem_amd.fingerprint import kernel_source_fingerprint  # noqa: E402

MARKER = "profile_marker_kernel"
CALIBRATION = "calibration"
CALIBRATION_KIB = float(1 << 20)   # 1 GiB in KiB, read and written
HBM_PEAK_GBS = 8000.0
# rows of the table of L1 requests in flight, in this order
INFLIGHT_WORKLOADS = ["put_block_256MiB_1blk", "put_block_256MiB_4blk", "put_block_256MiB_16blk", "get_block_256MiB_16blk",
                      "put_block_256MiB_filled", "stream_read_16blk", "stream_write_16blk", "stream_write_8blk", "stream_read_filled",
                      "stream_write_filled", "stream_write_through_filled", "reducescatter", "sum_reduce",
                      "alltoall_fp32_1GiB", "fcollect_int64", "broadcast", "moe_dispatch_put_signal", "moe_dispatch_plain_store",
                      "moe_combine", "calibration"]
INFLIGHT_TITLE = """L1-to-L2 requests a compute unit keeps in flight, by Little's law from the counters of ONE rocprofv3 pass
(TCP_TCC_READ_REQ, TCP_TCC_READ_REQ_LATENCY, TCP_TCC_WRITE_REQ, TCP_TCC_WRITE_REQ_LATENCY, GRBM_GUI_ACTIVE / 8 as the cycles):
in flight = requests x average latency / cycles / compute units occupied.  A read request is 128 bytes, a write
request 64.  "rd lat" / "wr lat" are average cycles per request, "sum" = reads + writes in flight, "KiB" their bytes.
Durations under the counter pass are a few percent longer than in the kernel trace; "kernel us" and GB/s
(algorithmic bytes per second) are the kernel trace's."""


COMMANDS = """Commands (on the GPU box, from the repository root; every file they run is committed):
  export OUT=<a scratch directory>; cd /tmp; export TMPDIR=/tmp
  export NVSHMEM_AMD_PLAIN_COLLECTIVE_LAUNCH=1   (kernels that nvshmemx_collective_launch starts are started with a plain
      launch: after a cooperative launch the profiled process crashes in an exit handler of the profiler's stack, behind
      the written results; the kernels and their grids are the same)
  rocprofv3 --kernel-trace --stats -d $OUT/stats -- python3 $REPO/nvshmem_amd/profile_workloads.py --iters 8 --manifest $OUT/manifest.json
  rocprofv3 --pmc FETCH_SIZE -d $OUT/p1 -- python3 $REPO/nvshmem_amd/profile_workloads.py --iters 8 --manifest $OUT/manifest.json
  rocprofv3 --pmc WRITE_SIZE -d $OUT/p2 -- (the same)
  rocprofv3 --pmc TCP_TCC_READ_REQ_sum TCP_TCC_READ_REQ_LATENCY_sum TCP_TCC_WRITE_REQ_sum TCP_TCC_WRITE_REQ_LATENCY_sum GRBM_GUI_ACTIVE -d $OUT/p3 -- (the same)
  rocprofv3 --pmc SQ_WAVES SQ_BUSY_CYCLES SQ_WAIT_INST_ANY SQ_INSTS_VMEM_RD SQ_INSTS_VMEM_WR SQ_INST_LEVEL_VMEM TCP_PENDING_STALL_CYCLES_sum TCP_TCR_TCP_STALL_CYCLES_sum -d $OUT/p4 -- (the same)
  rocprofv3 --pmc TCC_HIT_sum TCC_MISS_sum TCC_TAG_STALL_sum TCC_EA0_WRREQ_STALL_sum -d $OUT/p5 -- (the same)
  (every run must end with exit status 0)
  cd $REPO; python3 nvshmem_amd/profile_summary.py --manifest $OUT/manifest.json --stats $OUT/stats --pmc $OUT/p1 ... --pmc $OUT/p5 --profiles-dir profiles --inflight-table profiles/l1_requests_in_flight.txt
(a summary lists the counters of the passes that were run for it.)  Hardware: one MI355X (gfx950), ROCm 7.2.
Durations are per dispatch from the kernel trace."""


def _db(directory):
    hits = sorted(glob.glob(os.path.join(directory, "**", "*_results.db"), recursive=True), key=os.path.getmtime)
    if not hits:
        raise SystemExit("no *_results.db under %s" % directory)
    return sqlite3.connect(hits[-1])


def _short(name):
    name = name.replace("nvshmem_amd::(anonymous namespace)::", "").replace("(anonymous namespace)::", "")
    name = name.replace("void ", "")
    return name.split("(")[0]


def _windows(rows, manifest):
    """rows: (start, kernel name, payload...) of every dispatch -> {workload: [rows between its markers]}."""
    rows = sorted(rows, key=lambda r: r[0])
    out, index, inside = {}, -1, False
    for r in rows:
        if MARKER in r[1]:
            if not inside:
                index += 1
            inside = not inside
            continue
        if inside and 0 <= index < len(manifest):
            out.setdefault(manifest[index]["name"], []).append(r)
    return out


def kernel_windows(directory, manifest):
    cur = _db(directory).cursor()
    rows = cur.execute("select start, name, duration, grid_x, grid_y, grid_z, workgroup_x, vgpr_count from kernels").fetchall()
    return _windows([(s, _short(n), d, gx, gy, gz, wx, v) for s, n, d, gx, gy, gz, wx, v in rows], manifest)


def counter_windows(directory, manifest):
    cur = _db(directory).cursor()
    rows = cur.execute("select start, kernel_name, counter_name, value, dispatch_id from counters_collection").fetchall()
    # one row per (dispatch, counter); markers must be counted once per dispatch
    seen, flat = set(), []
    for s, n, c, v, d in rows:
        if MARKER in n:
            if d in seen:
                continue
            seen.add(d)
        flat.append((s, _short(n), c, v))
    return _windows(flat, manifest)


def stats_of(rows):
    """[(start, kernel, duration, grid...)] -> {kernel: (calls, avg us, min us, max us, launch shape, vgprs)}"""
    out = {}
    for _, k, d, gx, gy, gz, wx, v in rows:
        out.setdefault(k, []).append((d, (gx, gy, gz, wx), v))
    return {k: (len(v), sum(x[0] for x in v) / len(v) / 1e3, min(x[0] for x in v) / 1e3, max(x[0] for x in v) / 1e3,
                v[0][1], v[0][2]) for k, v in out.items()}


def counters_of(rows):
    """[(start, kernel, counter, value)] -> {kernel: {counter: average per dispatch}}"""
    acc = {}
    for _, k, c, v in rows:
        acc.setdefault(k, {}).setdefault(c, []).append(v)
    return {k: {c: sum(v) / len(v) for c, v in cs.items()} for k, cs in acc.items()}


def in_flight(cs, shape):
    """Little's law per compute unit: requests in flight = requests x latency / elapsed cycles, from the
    L1-to-L2 request and latency counters of one pass and GRBM_GUI_ACTIVE (which sums the busy cycles of
    the 8 XCDs).  shape = (grid threads x, y, z, block threads).  None when a counter is missing."""
    need = ("TCP_TCC_READ_REQ_LATENCY_sum", "TCP_TCC_WRITE_REQ_LATENCY_sum", "GRBM_GUI_ACTIVE")
    if any(k not in cs for k in need) or not cs["GRBM_GUI_ACTIVE"]:
        return None
    groups = shape[0] * shape[1] * shape[2] // max(1, shape[3])
    cus = min(groups, 256)
    cycles = cs["GRBM_GUI_ACTIVE"] / 8.0
    rr, wr = cs.get("TCP_TCC_READ_REQ_sum", 0), cs.get("TCP_TCC_WRITE_REQ_sum", 0)
    return {"groups": groups, "cus": cus, "cycles": cycles,
            "reads": cs["TCP_TCC_READ_REQ_LATENCY_sum"] / cycles / cus,
            "writes": cs["TCP_TCC_WRITE_REQ_LATENCY_sum"] / cycles / cus,
            "read_latency": cs["TCP_TCC_READ_REQ_LATENCY_sum"] / rr if rr else 0.0,
            "write_latency": cs["TCP_TCC_WRITE_REQ_LATENCY_sum"] / wr if wr else 0.0}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--manifest", required=True)
    ap.add_argument("--stats", required=True)
    ap.add_argument("--pmc", action="append", default=[])
    ap.add_argument("--profiles-dir")
    ap.add_argument("--only", default="")
    ap.add_argument("--table", default="", help="also write a one-line-per-workload table of the kernel trace there")
    ap.add_argument("--table-title", default="", help="first lines of that table")
    ap.add_argument("--inflight-table", default="", help="write the table of L1 requests in flight per compute unit there")
    args = ap.parse_args()
    manifest = json.load(open(args.manifest))
    only = set(x for x in args.only.split(",") if x)
    commands = COMMANDS
    kwin = kernel_windows(args.stats, manifest)
    cwins = [counter_windows(d, manifest) for d in args.pmc]
    # calibration factors
    scale = {}
    for cw in cwins:
        cal = counters_of(cw.get(CALIBRATION, []))
        for k, cs in cal.items():
            for c in ("FETCH_SIZE", "WRITE_SIZE"):
                if c in cs and cs[c] > 0:
                    scale[c] = CALIBRATION_KIB / cs[c]
    if args.table:
        rows = [args.table_title.replace("\\n", "\n"), "",
                "%-36s %-48s %6s %11s %11s %11s %8s %11s %9s" % ("workload", "dominant kernel", "calls", "avg us", "min us",
                                                                "max us", "kernels", "step us", "GB/s")]
        for entry in manifest:
            st = stats_of(kwin.get(entry["name"], []))
            if not st:
                continue
            k = max(st, key=lambda k: st[k][0] * st[k][1])
            calls, avg, lo, hi = st[k][:4]
            # a step may launch several kernels (a two-step allreduce, a dispatch with its signal kernel): the rate
            # is priced on the kernel time of the whole step
            step_us = sum(st[x][0] * st[x][1] for x in st) / max(1, entry["launches"])
            rows.append("%-36s %-48s %6d %11.2f %11.2f %11.2f %8d %11.2f %9.0f"
                        % (entry["name"], k[:48], calls, avg, lo, hi, len(st), step_us,
                           entry.get("algorithmic_bytes", 0) / step_us / 1e3))
        with open(args.table, "w") as fh:
            fh.write("\n".join(rows) + "\n")
    flight_rows = []
    for entry in manifest:
        name = entry["name"]
        if only and name not in only:
            continue
        st = stats_of(kwin.get(name, []))
        if not st:
            continue
        dominant = max(st, key=lambda k: st[k][0] * st[k][1])
        counters = {}
        for cw in cwins:
            for k, cs in counters_of(cw.get(name, [])).items():
                counters.setdefault(k, {}).update(cs)
        alg = entry.get("algorithmic_bytes", 2 << 30)
        lines = [entry.get("workload", "Counter calibration: plain one-vector-per-thread copy, 1 GiB read + 1 GiB written."),
                 "Algorithmic bytes per step: %d (%.1f MiB)." % (alg, alg / 2**20), ""]
        if commands:
            lines += [commands, ""]
        lines += ["%-58s %6s %11s %11s %11s  %s" % ("kernel", "calls", "avg us", "min us", "max us", "grid (threads) / block, VGPRs")]
        for k in sorted(st, key=lambda k: -st[k][0] * st[k][1]):
            calls, avg, lo, hi, shape, vg = st[k]
            lines.append("%-58s %6d %11.2f %11.2f %11.2f  %dx%dx%d / %d, %s" % (k[:58], calls, avg, lo, hi, shape[0], shape[1],
                                                                            shape[2], shape[3], vg))
        lines += ["", "kernel_sources_fingerprint: %s (nvshmem_amd/fingerprint.py, of the tree this was measured on)"
                  % kernel_source_fingerprint()]
        lines += ["", "dominant kernel: " + dominant]
        calls, avg = st[dominant][0], st[dominant][1]
        step_us = sum(st[k][0] * st[k][1] for k in st) / max(1, entry["launches"])
        lines.append("kernel time per step (all kernels of the step): %.2f us; dominant kernel alone: %.2f us per launch"
                     % (step_us, avg))
        # kernels that run once per step besides the dominant one and take a real share of it (the two kernels of a
        # two-step allreduce) make the step, not the dominant kernel, the unit of the rate
        shared = step_us > 1.25 * avg * calls / max(1, entry["launches"])
        unit_us = step_us if shared else avg
        lines.append("achieved = algorithmic bytes / %s = %.0f GB/s = %.1f %% of the %.0f GB/s HBM peak"
                     % ("kernel time of the step (several kernels share it)" if shared else "dominant kernel's average duration",
                        alg / unit_us / 1e3, alg / unit_us / 1e3 / HBM_PEAK_GBS * 100, HBM_PEAK_GBS))
        cs = counters.get(dominant, {})
        fl_row = in_flight(cs, st[dominant][4]) if cs else None
        if fl_row and name in INFLIGHT_WORKLOADS:
            flight_rows.append((name, dominant, st[dominant][1], alg / st[dominant][1] / 1e3, fl_row))  # single-kernel workloads
        if cs:
            lines += ["", "counters of the dominant kernel (average per dispatch):"]
            for c in sorted(cs):
                lines.append("  %-40s %18.1f" % (c, cs[c]))
            if "TCP_TCC_READ_REQ_LATENCY_sum" in cs and cs.get("TCP_TCC_READ_REQ_sum"):
                lines.append("  -> average L1-to-L2 read latency: %.0f cycles per request"
                             % (cs["TCP_TCC_READ_REQ_LATENCY_sum"] / cs["TCP_TCC_READ_REQ_sum"]))
            if "TCP_TCC_WRITE_REQ_LATENCY_sum" in cs and cs.get("TCP_TCC_WRITE_REQ_sum"):
                lines.append("  -> average L1-to-L2 write latency: %.0f cycles per request"
                             % (cs["TCP_TCC_WRITE_REQ_LATENCY_sum"] / cs["TCP_TCC_WRITE_REQ_sum"]))
            fl = in_flight(cs, st[dominant][4])
            if fl:
                lines.append("  -> %d work-groups on at most %d compute units, %.0f cycles: per compute unit on average %.1f L1 read "
                             "requests (128 bytes) and %.1f write requests (64 bytes) in flight, %.1f in all, %.1f KiB"
                             % (fl["groups"], fl["cus"], fl["cycles"], fl["reads"], fl["writes"], fl["reads"] + fl["writes"],
                                (128 * fl["reads"] + 64 * fl["writes"]) / 1024))
            if "TCC_EA0_RDREQ_LEVEL_sum" in cs and cs.get("TCC_EA0_RDREQ_sum"):
                lines.append("  -> average L2-to-fabric read latency: %.0f cycles per request"
                             % (cs["TCC_EA0_RDREQ_LEVEL_sum"] / cs["TCC_EA0_RDREQ_sum"]))
            if "TCC_HIT_sum" in cs and "TCC_MISS_sum" in cs and cs["TCC_HIT_sum"] + cs["TCC_MISS_sum"] > 0:
                lines.append("  -> L2 hit rate: %.1f %%" % (100 * cs["TCC_HIT_sum"] / (cs["TCC_HIT_sum"] + cs["TCC_MISS_sum"])))
            if "FETCH_SIZE" in cs and "WRITE_SIZE" in cs and "FETCH_SIZE" in scale and "WRITE_SIZE" in scale:
                if shared:      # the step's kernels together, each weighted by its launches per step
                    f = w = 0.0
                    for k in st:
                        per_step = st[k][0] / max(1, entry["launches"])
                        f += counters.get(k, {}).get("FETCH_SIZE", 0.0) * scale["FETCH_SIZE"] * 1024 * per_step
                        w += counters.get(k, {}).get("WRITE_SIZE", 0.0) * scale["WRITE_SIZE"] * 1024 * per_step
                    of_what = "step (all its kernels)"
                else:
                    f, w = cs["FETCH_SIZE"] * scale["FETCH_SIZE"] * 1024, cs["WRITE_SIZE"] * scale["WRITE_SIZE"] * 1024
                    of_what = "launch of the dominant kernel"
                lines += ["", "scale factors from the calibration copy (1 GiB read + 1 GiB written): FETCH_SIZE x%.4f, WRITE_SIZE x%.4f"
                          % (scale["FETCH_SIZE"], scale["WRITE_SIZE"]),
                          "measured_traffic_bytes: %d read + %d written = %.1f MiB per %s "
                          "(algorithmic %.1f MiB)" % (f, w, (f + w) / 2**20, of_what, alg / 2**20)]
        text = "\n".join(lines) + "\n"
        tag = re.split(r"[<(]", dominant)[0].strip().split("::")[-1]
        print("== %s (%s)" % (name, tag))
        print(text)
        if args.profiles_dir:
            os.makedirs(args.profiles_dir, exist_ok=True)
            for old in glob.glob(os.path.join(args.profiles_dir, "*__%s.txt" % name)):
                os.remove(old)
            with open(os.path.join(args.profiles_dir, "%s__%s.txt" % (tag, name)), "w") as fh:
                fh.write(text)


    if args.inflight_table and flight_rows:
        out = [INFLIGHT_TITLE, "", commands, "",
               "%-26s %5s %9s %8s | %8s %9s | %8s %9s | %7s %7s" % ("workload", "CUs", "kernel us", "GB/s", "rd lat", "rd in fl", "wr lat",
                                                                 "wr in fl", "sum", "KiB")]
        for name, kernel, us, gbs, fl in sorted(flight_rows, key=lambda r: INFLIGHT_WORKLOADS.index(r[0])):
            out.append("%-26s %5d %9.1f %8.0f | %8.0f %9.1f | %8.0f %9.1f | %7.1f %7.1f"
                       % (name, fl["cus"], us, gbs, fl["read_latency"], fl["reads"], fl["write_latency"], fl["writes"],
                          fl["reads"] + fl["writes"], (128 * fl["reads"] + 64 * fl["writes"]) / 1024))
        with open(args.inflight_table, "w") as fh:
            fh.write("\n".join(out) + "\n")


if __name__ == "__main__":
    main()
