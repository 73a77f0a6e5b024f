"""Summaries of rocprofv3 runs of bench.py, from the rocpd SQLite files rocprofv3 writes (`*_results.db`).

  python rocprof_summary.py trace <dir>
      per kernel and launch shape: calls, average / min / max duration in microseconds (a Markdown table)
  python rocprof_summary.py traffic <fetch_dir> <write_dir> [--kernel kq_gemv_many] [--json out.json]
      HBM bytes per launch of one kernel from two counter runs (`--pmc FETCH_SIZE`, `--pmc WRITE_SIZE`, KiB per
      dispatch), each scaled by what the same counter reads for the 256 MiB kq_copy_u128 of the same run; with --json the
      figure bench.py reports as `roofline.traffic` is written, stamped with the commit of the working tree.
  python rocprof_summary.py shapes <fetch_dir> <write_dir> [--prefix q4k_gemm]
      the same two counters per kernel and launch shape (a Markdown table): for kernels that serve several shapes
  python rocprof_summary.py runs <trace_dir> [<fetch_dir> <write_dir>] [--prefix q4k_gemm] [--min 100]
      runs of consecutive dispatches of one kernel and launch shape, in the order of the program (bench.py times a
      configuration as one such run: 20 + 5 x 200 launches over distinct copies, then as many on one copy): calls and
      average duration per run, with the two counters per run when their directories are given
  python rocprof_summary.py pmc <dir> [--prefix q4k_gemm] [--min 100]
      every counter of one `--pmc` run, averaged per dispatch over the same runs of consecutive dispatches
  python rocprof_summary.py timed <dir> --steps K [--ms-per-step T]
      the dispatches inside the regions bench.py brackets with a 4 KB kq_read_u128 (one workgroup): per region and kernel
      the calls, the average duration and the kernel time per pass (K passes to a region); with --ms-per-step the check that
      the kernel time per pass of the first region - the headline's - does not exceed what bench.py reported

The runs (on the GPU box, `cd /tmp && export TMPDIR=/tmp` first):
  rocprofv3 --kernel-trace --stats -d <dir> -- python3 bench.py --steps 20 --warmup 5 --pass-only
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
        root = os.path.dirname(os.path.abspath(__file__))
        result["commit"] = subprocess.run(["git", "-C", root, "rev-parse", "--short", "HEAD"], capture_output=True, text=True,
                                          check=True).stdout.strip()
    except Exception:
        result["commit"] = None
    print(json.dumps(result, indent=1))
    if json_out:
        with open(json_out, "w") as f:
            json.dump(result, f, indent=1)
            f.write("\n")


def shapes(fetch_dir: str, write_dir: str, prefix: str) -> None:
    def table(path, counter):
        out = {}
        for db in _dbs(path):
            con = sqlite3.connect(db)
            q = ("select kernel_name, grid_size_x, workgroup_size_x, avg(value), count(*) from counters_collection "
                 "where counter_name = ? group by kernel_name, grid_size_x, workgroup_size_x")
            for name, grid, wg, avg, n in con.execute(q, (counter,)):
                out[(name.split("(")[0], grid, wg)] = (float(avg), int(n))
        return out
    fetch, write = table(fetch_dir, "FETCH_SIZE"), table(write_dir, "WRITE_SIZE")
    copy_f = [v[0] for k, v in fetch.items() if k[0] == COPY_KERNEL]
    copy_w = [v[0] for k, v in write.items() if k[0] == COPY_KERNEL]
    if not copy_f or not copy_w:
        raise SystemExit(f"need a dispatch of {COPY_KERNEL} in both runs")
    scale_f, scale_w = COPY_KIB / copy_f[0], COPY_KIB / copy_w[0]
    print(f"scale: fetch {scale_f:.4f}, write {scale_w:.4f} ({COPY_KERNEL} over 256 MiB: FETCH_SIZE {copy_f[0]:.1f} KiB, WRITE_SIZE {copy_w[0]:.1f} KiB)")
    print("| kernel | grid threads | block | dispatches | FETCH KiB raw | WRITE KiB raw | HBM bytes (scaled) |")
    print("|---|---|---|---|---|---|---|")
    for key in sorted(fetch):
        if not key[0].startswith(prefix) or key not in write:
            continue
        f, w = fetch[key], write[key]
        print(f"| {key[0]} | {key[1]} | {key[2]} | {f[1]} | {f[0]:.1f} | {w[0]:.1f} | {round((f[0] * scale_f + w[0] * scale_w) * 1024):,} |")


def _runs(path: str, query: str, prefix: str):
    """[(key, [values])] for consecutive rows with the same key = (kernel, grid, block)"""
    out = []
    for db in _dbs(path):
        con = sqlite3.connect(db)
        for name, grid, wg, value in con.execute(query):
            key = (name.split("(")[0], grid, wg)
            if out and out[-1][0] == key:
                out[-1][1].append(float(value))
            else:
                out.append((key, [float(value)]))
    return [(k, v) for k, v in out if k[0].startswith(prefix)]


def runs(trace_dir: str, fetch_dir: str | None, write_dir: str | None, prefix: str, least: int) -> None:
    tr = [r for r in _runs(trace_dir, "select name, grid_x, workgroup_x, end - start from kernels order by start", prefix)
          if len(r[1]) >= least]
    cols = [tr]
    if fetch_dir and write_dir:
        q = ("select kernel_name, grid_size_x, workgroup_size_x, value from counters_collection where counter_name = '{}' "
             "order by dispatch_id")
        fetch = [r for r in _runs(fetch_dir, q.format("FETCH_SIZE"), prefix) if len(r[1]) >= least]
        write = [r for r in _runs(write_dir, q.format("WRITE_SIZE"), prefix) if len(r[1]) >= least]
        if [r[0] for r in fetch] != [r[0] for r in tr] or [r[0] for r in write] != [r[0] for r in tr]:
            raise SystemExit("the three runs do not show the same sequence of kernel runs")
        copy_f = _runs(fetch_dir, q.format("FETCH_SIZE"), COPY_KERNEL)[0][1][0]
        copy_w = _runs(write_dir, q.format("WRITE_SIZE"), COPY_KERNEL)[0][1][0]
        print(f"scale: fetch {COPY_KIB / copy_f:.4f}, write {COPY_KIB / copy_w:.4f}")
        cols += [fetch, write, COPY_KIB / copy_f, COPY_KIB / copy_w]
    head = "| # | kernel | grid threads | block | calls | average us | min us |"
    print(head + (" FETCH KiB raw | WRITE KiB raw | HBM bytes (scaled) |" if len(cols) > 1 else ""))
    print("|---" * (head.count("|") - 1 + (3 if len(cols) > 1 else 0)) + "|")
    for i, (key, d) in enumerate(tr):
        line = f"| {i} | {key[0]} | {key[1]} | {key[2]} | {len(d)} | {sum(d) / len(d) / 1e3:.2f} | {min(d) / 1e3:.2f} |"
        if len(cols) > 1:
            f, w = cols[1][i][1], cols[2][i][1]
            fa, wa = sum(f) / len(f), sum(w) / len(w)
            line += f" {fa:.1f} | {wa:.1f} | {round((fa * cols[3] + wa * cols[4]) * 1024):,} |"
        print(line)


def pmc(path: str, prefix: str, least: int) -> None:
    names = []
    for db in _dbs(path):
        names += [r[0] for r in sqlite3.connect(db).execute("select distinct counter_name from counters_collection order by 1")]
    names = sorted(set(names))
    q = ("select kernel_name, grid_size_x, workgroup_size_x, value from counters_collection where counter_name = '{}' "
         "order by dispatch_id")
    tables = [[r for r in _runs(path, q.format(n), prefix) if len(r[1]) >= least] for n in names]
    print("| # | kernel | grid threads | block | calls | " + " | ".join(names) + " |")
    print("|---" * (5 + len(names)) + "|")
    for i, (key, d) in enumerate(tables[0]):
        vals = " | ".join(f"{sum(t[i][1]) / len(t[i][1]):,.0f}" for t in tables)
        print(f"| {i} | {key[0]} | {key[1]} | {key[2]} | {len(d)} | {vals} |")


def timed(path: str, steps: int, ms_per_step: float | None) -> None:
    for db in _dbs(path):
        con = sqlite3.connect(db)
        rows = list(con.execute("select name, grid_x, workgroup_x, start, end from kernels order by start"))
        marks = [i for i, r in enumerate(rows) if r[0].split("(")[0] == "kq_read_u128" and r[1] == 256]
        if len(marks) < 2:
            raise SystemExit("no pair of region marks (kq_read_u128 over 4 KB) in the trace")
        for region in range(len(marks) // 2):
            inside = rows[marks[2 * region] + 1:marks[2 * region + 1]]
            by = {}
            for name, grid, wg, start, end in inside:
                by.setdefault((name.split("(")[0], grid, wg), []).append((end - start) / 1e3)
            # the warm-up passes of a region come before its first mark only in the headline region; a region's first
            # `len - steps * calls_per_pass` dispatches would be warm-up otherwise: bench.py marks after the warm-up
            span = (inside[-1][4] - inside[0][3]) / 1e3 if inside else 0.0
            total = sum(sum(v) for v in by.values())
            print(f"region {region}: {len(inside)} dispatches, first start to last end {span / steps:.1f} us per pass, "
                  f"kernel time {total / steps:.1f} us per pass")
            print("| kernel | grid threads | block | calls | calls per pass | average us | min us | max us | us per pass |")
            print("|---|---|---|---|---|---|---|---|---|")
            for key, v in sorted(by.items(), key=lambda kv: -sum(kv[1])):
                print(f"| {key[0]} | {key[1]} | {key[2]} | {len(v)} | {len(v) / steps:g} | {sum(v) / len(v):.2f} | {min(v):.2f} | {max(v):.2f} | {sum(v) / steps:.1f} |")
            if region == 0 and ms_per_step is not None:
                ok = total / steps <= ms_per_step * 1e3
                print(f"check: kernel time per pass {total / steps:.1f} us {'<=' if ok else '>'} ms_per_step {ms_per_step * 1e3:.1f} us: {'holds' if ok else 'FAILS'}")


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    tr = sub.add_parser("trace")
    tr.add_argument("dir")
    tf = sub.add_parser("traffic")
    tf.add_argument("fetch_dir")
    tf.add_argument("write_dir")
    tf.add_argument("--kernel", default="kq_gemv_many")
    tf.add_argument("--json")
    sh = sub.add_parser("shapes")
    sh.add_argument("fetch_dir")
    sh.add_argument("write_dir")
    sh.add_argument("--prefix", default="")
    rn = sub.add_parser("runs")
    rn.add_argument("trace_dir")
    rn.add_argument("fetch_dir", nargs="?")
    rn.add_argument("write_dir", nargs="?")
    rn.add_argument("--prefix", default="")
    rn.add_argument("--min", type=int, default=100)
    pm = sub.add_parser("pmc")
    pm.add_argument("dir")
    pm.add_argument("--prefix", default="")
    pm.add_argument("--min", type=int, default=100)
    tm = sub.add_parser("timed")
    tm.add_argument("dir")
    tm.add_argument("--steps", type=int, required=True)
    tm.add_argument("--ms-per-step", type=float)
    a = ap.parse_args()
    if a.cmd == "timed":
        timed(a.dir, a.steps, a.ms_per_step)
    elif a.cmd == "trace":
        trace(a.dir)
    elif a.cmd == "pmc":
        pmc(a.dir, a.prefix, a.min)
    elif a.cmd == "runs":
        runs(a.trace_dir, a.fetch_dir, a.write_dir, a.prefix, a.min)
    elif a.cmd == "shapes":
        shapes(a.fetch_dir, a.write_dir, a.prefix)
    else:
        traffic(a.fetch_dir, a.write_dir, a.kernel, a.json)
    return 0


if __name__ == "__main__":
    sys.exit(main())
