"""Turn the CSV that ``rocprofv3 --kernel-trace --stats`` writes into the short
text summary kept under ``profiles/``.

    python -m ssm_amd.profile_summary <dir-with-*_kernel_stats.csv> "<command that was profiled>"
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


if __name__ == "__main__":
    sys.stdout.write(summarise(sys.argv[1], sys.argv[2] if len(sys.argv) > 2 else "?"))
