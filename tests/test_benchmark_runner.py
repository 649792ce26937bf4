"""The profiler-wrapping benchmark runner (fusilli_amd/bench/run_benchmark.py),
counterpart of the reference's benchmarks/run_benchmark.py: trace parsing and
grouping on the CPU with a synthetic trace, and the contract of the reference's
benchmarks/test_benchmark_runner.sh:22-43 on the GPU (one row per command,
`iter` and `dispatch_count` columns, iter = 2)."""
import csv
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "fusilli_amd", "bench")
sys.path.insert(0, BENCH)
import run_benchmark as rb  # noqa: E402


def _write_trace(path, durations_ns, extra_rows=()):
    with open(path, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["Kind", "Agent_Id", "Kernel_Name", "Start_Timestamp",
                    "End_Timestamp"])
        t = 1000
        rows = []
        for d in durations_ns:
            rows.append(["KERNEL_DISPATCH", "1", "k", str(t), str(t + d)])
            t += d + 500
        rows = rows[::-1]  # file order is not start order
        for r in list(extra_rows) + rows:
            w.writerow(r)


def test_trace_is_grouped_into_iterations(tmp_path):
    # 3 warm-up + 4 timed iterations of 2 kernels each
    durs = [9000, 9000] * 3 + [1000, 2000, 1500, 2500, 1000, 1000, 3000, 1000]
    sub = tmp_path / "host" / "123"
    sub.mkdir(parents=True)
    _write_trace(sub / "123_kernel_trace.csv", durs,
                 extra_rows=[["MEMORY_COPY", "1", "", "10", "20"],
                            ["KERNEL_DISPATCH", "1",
                             "__amd_rocclr_copyBuffer.kd", "30", "40"]])
    got = rb.kernel_durations_us(tmp_path)
    assert got == [d / 1000.0 for d in durs]
    st = rb.iteration_stats(got, iters=4, warmup=3)
    assert (st.iter, st.dispatch_count) == (4, 2)
    assert st.min == 2.0 and st.max == 4.0 and st.mean == pytest.approx(3.25)
    assert st.stddev == pytest.approx(0.9574, abs=1e-3)


def test_trace_that_does_not_divide_is_an_error(tmp_path):
    with pytest.raises(RuntimeError):
        rb.iteration_stats([1.0] * 7, iters=2, warmup=3)
    assert rb.iteration_stats([], iters=2, warmup=3) == rb.Stats()


def test_skip_and_missing_driver_rows(tmp_path):
    cmds = tmp_path / "cmds.txt"
    cmds.write_text("# comment\n[SKIP] --iter 2 matmul -M 1\n--iter 2 matmul -M 1\n")
    out = tmp_path / "out.csv"
    rc = rb.main(["-f", str(cmds), "-o", str(out), "-D",
                  str(tmp_path / "no_such_driver"), "-t", "20"])
    rows = list(csv.reader(open(out)))
    assert rc == 1  # the second command cannot run
    assert rows[0] == ["command", "min (us)", "max (us)", "mean (us)",
                       "stddev (us)", "iter", "dispatch_count"]
    assert len(rows) == 3 and rows[1][1:] == ["N.A."] * 6


@pytest.mark.gpu
def test_runner_contract_on_reference_test_commands(tmp_path):
    # the four commands of the reference's benchmarks/test_commands.txt
    src = [l.strip() for l in open(os.path.join(BENCH, "test_commands.txt"))
           if l.strip() and not l.startswith("#")][:4]
    cmds = tmp_path / "cmds.txt"
    cmds.write_text("\n".join(src) + "\n")
    out = tmp_path / "out.csv"
    proc = subprocess.run(
        [sys.executable, os.path.join(BENCH, "run_benchmark.py"), "-f", str(cmds),
         "-o", str(out), "--verbose", "-t", "120"],
        capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-2000:]
    rows = list(csv.DictReader(open(out)))
    assert len(rows) == len(src)
    for r in rows:
        assert r["iter"] == "2" and r["dispatch_count"] == "1"
        assert 0 < float(r["min (us)"]) <= float(r["mean (us)"]) <= float(r["max (us)"])


def test_bench_refuses_more_than_one_gpu():
    # bench.py measures one GPU; a multi-GPU request ends before anything is
    # loaded, with a message that says so
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)
