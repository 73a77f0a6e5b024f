"""The profiler summaries (rocprof_summary.py) on a hand-made trace database: the timed region is what lies between two
region marks, its kernel time per pass is checked against the benchmark's own figure, and the per-shape table groups by
kernel and launch shape."""
import importlib.util
import os
import sqlite3

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("rocprof_summary", os.path.join(ROOT, "rocprof_summary.py"))
rocprof_summary = importlib.util.module_from_spec(spec)
spec.loader.exec_module(rocprof_summary)

MARK = ("kq_read_u128(uint4 const*, unsigned long, unsigned int*)", 256, 256)
MANY = ("kq_gemv_many", 196608, 768)
HEAD = ("kq_gemv_group", 130048, 512)


def _trace(tmp_path, launches):
    """launches: [(name, grid, block, duration in ns)], laid out back to back with gaps of 1 us"""
    d = tmp_path / "out" / "vm"
    d.mkdir(parents=True)
    con = sqlite3.connect(str(d / "1_results.db"))
    con.execute("create table kernels (name text, grid_x int, workgroup_x int, start int, end int)")
    t = 1000
    for name, grid, block, ns in launches:
        con.execute("insert into kernels values (?, ?, ?, ?, ?)", (name, grid, block, t, t + ns))
        t += ns + 1000
    con.commit()
    con.close()
    return str(tmp_path / "out")


def test_timed_region_is_what_lies_between_two_marks(tmp_path, capsys):
    warm = [(*MANY, 500_000), (*MANY, 400_000), (*HEAD, 40_000)]                    # before the first mark: not counted
    one_pass = [(*MANY, 400_000), (*MANY, 300_000), (*HEAD, 25_000)]
    path = _trace(tmp_path, warm + [(*MARK, 2000)] + one_pass * 2 + [(*MARK, 2000)] + [(*MANY, 999_000)])
    rocprof_summary.timed(path, 2, 0.730)
    out = capsys.readouterr().out
    assert "region 0: 6 dispatches" in out and "kernel time 725.0 us per pass" in out
    assert "| kq_gemv_many | 196608 | 768 | 4 | 2 | 350.00 | 300.00 | 400.00 | 700.0 |" in out
    assert "| kq_gemv_group | 130048 | 512 | 2 | 1 | 25.00 | 25.00 | 25.00 | 25.0 |" in out
    assert "check: kernel time per pass 725.0 us <= ms_per_step 730.0 us: holds" in out
    assert "999" not in out                                                          # behind the second mark: not counted


def test_timed_check_fails_when_the_kernels_took_longer_than_reported(tmp_path, capsys):
    path = _trace(tmp_path, [(*MARK, 2000), (*MANY, 400_000), (*MANY, 300_000), (*MARK, 2000)])
    rocprof_summary.timed(path, 1, 0.650)
    assert "FAILS" in capsys.readouterr().out


def test_trace_groups_by_kernel_and_launch_shape(tmp_path, capsys):
    path = _trace(tmp_path, [(*MANY, 400_000), (*MANY, 300_000), (*HEAD, 25_000), (*MARK, 2000)])
    rocprof_summary.trace(path)
    out = capsys.readouterr().out
    assert "| kq_gemv_many | 196608 | 768 | 2 | 350.00 | 300.00 | 400.00 |" in out
    assert "| kq_read_u128 | 256 | 256 | 1 | 2.00 | 2.00 | 2.00 |" in out
