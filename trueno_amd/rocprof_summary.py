"""Summaries of rocprofv3 runs of bench.py, from the rocpd SQLite files rocprofv3 writes (`*_results.db`).

  python -m trueno_amd.rocprof_summary trace <dir>
      per kernel and launch shape: calls, average / min / max duration in microseconds (a Markdown table)
  python -m trueno_amd.rocprof_summary traffic <fetch_dir> <write_dir> [--kernel kq_gemv_group] [--json out.json]
      HBM bytes per launch of one kernel from two counter runs (`--pmc FETCH_SIZE`, `--pmc WRITE_SIZE`, KiB per
      dispatch), each scaled by what the same counter reads for the 256 MiB kq_copy_u128 of the same run; with --json the
      figure bench.py reports as `roofline.traffic` is written, stamped with the commit of the working tree.

The runs (on the GPU box, `cd /tmp && export TMPDIR=/tmp` first):
  rocprofv3 --kernel-trace --stats -d <dir> -- python3 bench.py --steps 10 --warmup 2 --no-cpu-baseline --no-executors --no-configs
  rocprofv3 --pmc FETCH_SIZE -d <fetch_dir> -- python3 bench.py --steps 2 --warmup 1 --pass-only
  rocprofv3 --pmc WRITE_SIZE -d <write_dir> -- python3 bench.py --steps 2 --warmup 1 --pass-only
"""
from __future__ import annotations

import argparse
import glob
import json
import os
import sqlite3
import subprocess
import sys

COPY_KERNEL, COPY_KIB = "kq_copy_u128", 262144.0      # bench.py copies 256 MiB once: that much read, that much written


def _dbs(path: str):
    found = sorted(glob.glob(os.path.join(path, "**", "*_results.db"), recursive=True))
    if not found:
        raise SystemExit(f"no *_results.db under {path}")
    return found


def trace(path: str) -> None:
    print("| kernel | grid threads | block | calls | average us | min us | max us |")
    print("|---|---|---|---|---|---|---|")
    for db in _dbs(path):
        con = sqlite3.connect(db)
        q = ("select name, grid_x, workgroup_x, count(*), avg(end - start), min(end - start), max(end - start) from kernels "
             "group by name, grid_x, workgroup_x order by sum(end - start) desc")
        for name, grid, wg, calls, avg, lo, hi in con.execute(q):
            print(f"| {name.split('(')[0]} | {grid} | {wg} | {calls} | {avg / 1e3:.2f} | {lo / 1e3:.2f} | {hi / 1e3:.2f} |")


def _counter(path: str, counter: str):
    """{kernel: (average value, dispatches)} of one counter"""
    out = {}
    for db in _dbs(path):
        con = sqlite3.connect(db)
        q = "select kernel_name, avg(value), count(*) from counters_collection where counter_name = ? group by kernel_name"
        for name, avg, n in con.execute(q, (counter,)):
            out[name.split("(")[0]] = (float(avg), int(n))
    return out


def traffic(fetch_dir: str, write_dir: str, kernel: str, json_out: str | None) -> None:
    fetch, write = _counter(fetch_dir, "FETCH_SIZE"), _counter(write_dir, "WRITE_SIZE")
    for name, table in (("FETCH_SIZE", fetch), ("WRITE_SIZE", write)):
        if COPY_KERNEL not in table or kernel not in table:
            raise SystemExit(f"{name}: need dispatches of {COPY_KERNEL} and {kernel}, found {sorted(table)}")
    scale_f, scale_w = COPY_KIB / fetch[COPY_KERNEL][0], COPY_KIB / write[COPY_KERNEL][0]
    fetch_b, write_b = fetch[kernel][0] * scale_f * 1024.0, write[kernel][0] * scale_w * 1024.0
    result = {"kernel": kernel, "bytes_per_launch": round(fetch_b + write_b), "fetch_bytes_per_launch": round(fetch_b),
              "write_bytes_per_launch": round(write_b), "dispatches": fetch[kernel][1],
              "fetch_size_kib_raw": round(fetch[kernel][0], 1), "write_size_kib_raw": round(write[kernel][0], 1),
              "scale_fetch": round(scale_f, 4), "scale_write": round(scale_w, 4),
              "yardstick": f"{COPY_KERNEL} over 256 MiB reads FETCH_SIZE {fetch[COPY_KERNEL][0]:.1f} KiB, WRITE_SIZE {write[COPY_KERNEL][0]:.1f} KiB",
              "command": "rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE -d <dir> -- python3 bench.py --steps 2 --warmup 1 --pass-only"}
    try:
        root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
        result["commit"] = subprocess.run(["git", "-C", root, "rev-parse", "--short", "HEAD"], capture_output=True, text=True,
                                          check=True).stdout.strip()
    except Exception:
        result["commit"] = None
    print(json.dumps(result, indent=1))
    if json_out:
        with open(json_out, "w") as f:
            json.dump(result, f, indent=1)
            f.write("\n")


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    tr = sub.add_parser("trace")
    tr.add_argument("dir")
    tf = sub.add_parser("traffic")
    tf.add_argument("fetch_dir")
    tf.add_argument("write_dir")
    tf.add_argument("--kernel", default="kq_gemv_group")
    tf.add_argument("--json")
    a = ap.parse_args()
    if a.cmd == "trace":
        trace(a.dir)
    else:
        traffic(a.fetch_dir, a.write_dir, a.kernel, a.json)
    return 0


if __name__ == "__main__":
    sys.exit(main())
