"""Summaries of `rocprofv3 --pmc` counter output for the benchmark kernels.

    python -m t2sp_amd.pmc_summary --fetch DIR --write DIR [--kernel SUBSTRING] [--out FILE]

DIR are the output directories of two counter runs of bench.py (one counter per run):

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d DIR_F -o f -- python3 bench.py --steps 3 --warmup 1 --no-cpu --no-others --calibrate-copy
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d DIR_W -o w -- python3 bench.py --steps 3 --warmup 1 --no-cpu --no-others --calibrate-copy

`--calibrate-copy` makes bench.py run a plain copy of 64 Mi floats first; what FETCH_SIZE and WRITE_SIZE
read for that copy (256 MiB each way) gives the factor each counter is scaled by.  The table of every
kernel goes to stdout; with --out, the figures of the kernel whose name contains SUBSTRING (default: the
LDS-tiled SGEMM kernel, which with --no-others only runs the 8192^3 headline) are written as
`key value` lines, the file bench.py reads its roofline.traffic from.
"""
import argparse
import csv
import glob
import os
import sys
from collections import defaultdict

COPY_KIB = 64 * 1024 * 1024 * 4 / 1024.0      # the calibration copy moves this much each way
COPY_GRID = 16777216                          # and is launched with this many threads


def per_kernel(directory, counter):
    """{kernel name: (launches, mean counter value per launch)} and the calibration copy's mean."""
    files = glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise SystemExit("no *counter_collection.csv under %s" % directory)
    acc, copy = defaultdict(list), []
    for f in files:
        for row in csv.DictReader(open(f, newline="")):
            if row["Counter_Name"] != counter:
                continue
            name, value = row["Kernel_Name"], float(row["Counter_Value"])
            if "relayout_kernel" in name and int(row["Grid_Size"]) == COPY_GRID:
                copy.append(value)
            else:
                acc[name].append(value)
    if not copy:
        raise SystemExit("no calibration copy in %s: run bench.py with --calibrate-copy" % directory)
    return {k: (len(v), sum(v) / len(v)) for k, v in acc.items()}, sum(copy) / len(copy)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--fetch", required=True)
    ap.add_argument("--write", required=True)
    ap.add_argument("--kernel", default="sgemm_kernel<")
    ap.add_argument("--out")
    a = ap.parse_args()
    fetch, copy_f = per_kernel(a.fetch, "FETCH_SIZE")
    write, copy_w = per_kernel(a.write, "WRITE_SIZE")
    fs, ws = COPY_KIB / copy_f, COPY_KIB / copy_w
    print("calibration copy: FETCH_SIZE %.1f KiB, WRITE_SIZE %.1f KiB per 262144 KiB each way -> scale %.3f / %.3f" % (
        copy_f, copy_w, fs, ws))
    print("| kernel | launches | FETCH_SIZE KiB (raw avg) | WRITE_SIZE KiB (raw avg) | scaled read MB | scaled write MB |")
    print("|---|---|---|---|---|---|")
    for name in sorted(fetch):
        if not name.startswith("t2sp::") and "t2sp" not in name:
            continue
        n, f = fetch[name]
        w = write.get(name, (0, 0.0))[1]
        print("| `%s` | %d | %.1f | %.1f | %.1f | %.1f |" % (name[:110], n, f, w, f * fs * 1024 / 1e6, w * ws * 1024 / 1e6))
    if a.out:
        pick = [k for k in fetch if a.kernel in k]
        if len(pick) != 1:
            raise SystemExit("--kernel %r matches %d kernels: %s" % (a.kernel, len(pick), pick))
        (n, f), w = fetch[pick[0]], write[pick[0]][1]
        with open(a.out, "w") as fp:
            fp.write("# HBM-side traffic of one launch of the kernel below, from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE),\n"
                     "# each scaled by what the same counter reads for a 256 MiB copy.  Written by: %s\n" % " ".join(
                         ["python", "-m", "t2sp_amd.pmc_summary"] + sys.argv[1:]))
            fp.write("kernel %s\nlaunches %d\nfetch_kib_raw %.1f\nwrite_kib_raw %.1f\nfetch_scale %.3f\nwrite_scale %.3f\n" % (
                pick[0], n, f, w, fs, ws))
            fp.write("traffic_bytes %.4g\n" % ((f * fs + w * ws) * 1024))
        print("wrote", a.out)


if __name__ == "__main__":
    main()
