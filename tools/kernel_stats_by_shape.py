"""Per-kernel launch times of a `rocprofv3 --kernel-trace --output-format csv` run, grouped by kernel AND launch shape (the same kernel
serves prompts and single tokens: one average over both says nothing).

    python tools/kernel_stats_by_shape.py <dir or *_kernel_trace.csv> [min_calls] > profiles/<name>_kernel_stats_by_launch_shape.txt
"""
import csv
import glob
import os
import re
import sys


def main():
    src = sys.argv[1]
    min_calls = int(sys.argv[2]) if len(sys.argv) > 2 else 1
    files = [src] if os.path.isfile(src) else glob.glob(os.path.join(src, "**", "*kernel_trace.csv"), recursive=True)
    stats = {}
    for f in files:
        with open(f, newline="") as fh:
            for row in csv.DictReader(fh):
                name = re.sub(r"^void ", "", row["Kernel_Name"])
                name = re.sub(r"\(anonymous namespace\)::", "", name)
                name = re.sub(r"\(.*$", "", name)
                wg = [int(row[k]) for k in ("Workgroup_Size_X", "Workgroup_Size_Y", "Workgroup_Size_Z")]
                grid = [int(row[k]) // max(w, 1) for k, w in zip(("Grid_Size_X", "Grid_Size_Y", "Grid_Size_Z"), wg)]
                key = (name, "(%d,%d,%d)/%d" % (grid[0], grid[1], grid[2], wg[0] * wg[1] * wg[2]))
                us = (int(row["End_Timestamp"]) - int(row["Start_Timestamp"])) / 1e3
                s = stats.setdefault(key, [0, 0.0, 1e30, 0.0])
                s[0] += 1
                s[1] += us
                s[2] = min(s[2], us)
                s[3] = max(s[3], us)
    print("%-60s %-28s %7s %9s %9s %9s" % ("kernel", "grid (workgroups) / threads", "calls", "avg_us", "min_us", "max_us"))
    for (name, shape), s in sorted(stats.items()):
        if s[0] >= min_calls:
            print("%-60s %-28s %7d %9.1f %9.1f %9.1f" % (name[:60], shape, s[0], s[1] / s[0], s[2], s[3]))


if __name__ == "__main__":
    main()
