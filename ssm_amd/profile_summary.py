"""Turn the CSV files that ``rocprofv3`` writes into the short text summaries kept
under ``profiles/``.

    python -m ssm_amd.profile_summary <dir-with-*_kernel_stats.csv> "<command that was profiled>"
    python -m ssm_amd.profile_summary --pmc <dir-with-*_counter_collection.csv> "<command>"

The second form averages every hardware counter per kernel over its dispatches
(``rocprofv3 --pmc`` output).
"""

from __future__ import annotations

import csv
import glob
import sys


def summarise(folder: str, command: str, top: int = 25) -> str:
    files = glob.glob(f"{folder}/**/*kernel_stats.csv", recursive=True)
    if not files:
        raise SystemExit(f"no *kernel_stats.csv under {folder}")
    rows = list(csv.DictReader(open(files[0])))
    rows.sort(key=lambda r: -float(r["TotalDurationNs"]))
    out = [f"command: {command}", f"source:  {files[0].split('/')[-1]} (rocprofv3 --kernel-trace --stats)", "",
           f"{'kernel':<96} {'calls':>6} {'avg_us':>10} {'min_us':>10} {'max_us':>10} {'pct':>6}"]
    for r in rows[:top]:
        name = r["Name"]
        name = name if len(name) <= 95 else name[:92] + "..."
        out.append(f"{name:<96} {int(r['Calls']):>6} {float(r['AverageNs']) / 1e3:>10.2f} "
                   f"{float(r['MinNs']) / 1e3:>10.2f} {float(r['MaxNs']) / 1e3:>10.2f} {float(r['Percentage']):>6.2f}")
    return "\n".join(out) + "\n"


def summarise_pmc(folder: str, command: str) -> str:
    files = glob.glob(f"{folder}/**/*counter_collection.csv", recursive=True)
    if not files:
        raise SystemExit(f"no *counter_collection.csv under {folder}")
    acc = {}
    for r in csv.DictReader(open(files[0])):
        acc.setdefault((r["Kernel_Name"], r["Counter_Name"]), []).append(float(r["Counter_Value"]))
    out = [f"command: {command}", f"source:  {files[0].split('/')[-1]} (rocprofv3 --pmc)", "",
           f"{'kernel':<96} {'counter':<24} {'dispatches':>10} {'mean per dispatch':>20}"]
    for (name, counter), vals in sorted(acc.items(), key=lambda kv: (-sum(kv[1]), kv[0])):
        name = name if len(name) <= 95 else name[:92] + "..."
        out.append(f"{name:<96} {counter:<24} {len(vals):>10} {sum(vals) / len(vals):>20.1f}")
    return "\n".join(out) + "\n"


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "--pmc":
        sys.stdout.write(summarise_pmc(sys.argv[2], sys.argv[3] if len(sys.argv) > 3 else "?"))
    else:
        sys.stdout.write(summarise(sys.argv[1], sys.argv[2] if len(sys.argv) > 2 else "?"))
