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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--stats", required=True)
    ap.add_argument("--fetch")
    ap.add_argument("--write")
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


if __name__ == "__main__":
    main()
