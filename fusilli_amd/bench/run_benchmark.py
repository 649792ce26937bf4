#!/usr/bin/env python3
"""Profiler-derived per-iteration kernel times for the benchmark driver.

The counterpart of the reference's benchmarks/run_benchmark.py (:41-119 trace
parsing, :120-216 one profiled command, :219-441 command-line interface and the
result table; its contract: benchmarks/test_benchmark_runner.sh:22-43).  Every
command of a commands file (one per line, `#` comments, `[SKIP]` prefix) is run
as a fresh child process

    rocprofv3 --output-format csv --output-directory <dir> --kernel-trace -- <driver> <args>

and the kernel dispatches of its `*kernel_trace.csv` are grouped into the
driver's `--iter` iterations: the time of an iteration is the sum of the
durations of the kernels it launched.  One row per command goes into the
result CSV:

    command, min (us), max (us), mean (us), stddev (us), iter, dispatch_count

This process never touches the GPU itself.  Differences from the reference's
runner: kernels are recognised by the trace's dispatch rows (minus the HIP
runtime's own copy kernels) rather than by the `async_dispatch` substring of
IREE's kernel names; the driver's untimed warm-up
executes (`--warmup`, 3 by default) are dropped from the front of the trace;
`--knob NAME=VALUE` (repeatable) sets a FUSILLI_HIP_<NAME> tuning variable for
the driver where the reference forwards `--Xiree-compile` flags to its compiler.
"""
from __future__ import annotations

import argparse
import csv
import os
import shlex
import statistics
import subprocess
import sys
import tempfile
from pathlib import Path
from typing import List, NamedTuple, Optional, Union

Number = Union[float, int, str]
METRICS = ["min", "max", "mean", "stddev", "iter", "dispatch_count"]
NA = "N.A."
DRIVER_WARMUP = 3  # untimed executes the driver runs before its --iter loop


class Stats(NamedTuple):
    min: Number = NA
    max: Number = NA
    mean: Number = NA
    stddev: Number = NA
    iter: Number = NA
    dispatch_count: Number = NA


def kernel_durations_us(trace_dir: Path) -> List[float]:
    """Durations of all kernel dispatches under `trace_dir`, in start order."""
    rows = []
    for path in sorted(trace_dir.rglob("*kernel_trace.csv")):
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if "Start_Timestamp" not in row or "End_Timestamp" not in row:
                    continue
                kind = row.get("Kind", "KERNEL_DISPATCH")
                if "KERNEL_DISPATCH" not in kind.upper():
                    continue
                # the HIP runtime's own copy / fill kernels (small host-to-
                # device uploads of the inputs run as such) are not the graph's
                if row.get("Kernel_Name", "").startswith("__amd_rocclr_"):
                    continue
                start, end = float(row["Start_Timestamp"]), float(row["End_Timestamp"])
                rows.append((start, (end - start) / 1000.0))
    rows.sort()
    return [d for _, d in rows]


def iteration_stats(durations: List[float], iters: int, warmup: int) -> Stats:
    """Groups consecutive dispatches into warmup + iters equal iterations and
    returns the statistics of the timed ones."""
    if not durations:
        return Stats()
    total = len(durations)
    groups = iters + warmup
    if iters <= 0 or total < groups or total % groups != 0:
        raise RuntimeError(
            f"{total} kernel dispatches do not divide into {warmup} warm-up + "
            f"{iters} timed iterations")
    per_iter = total // groups
    sums = [sum(durations[i * per_iter:(i + 1) * per_iter])
            for i in range(warmup, groups)]
    return Stats(min=min(sums), max=max(sums), mean=statistics.mean(sums),
                 stddev=statistics.stdev(sums) if len(sums) > 1 else 0.0,
                 iter=len(sums), dispatch_count=per_iter)


def option_value(args: List[str], names, default: int) -> int:
    for name in names:
        if name in args and args.index(name) + 1 < len(args):
            return int(args[args.index(name) + 1])
    return default


def run_profiled(command: str, driver: str, out_dir: Optional[Path],
                 rocprof_args: List[str], env: dict, verbose: bool, number: int,
                 timeout: Optional[int]):
    """Returns (Stats, outcome) with outcome in ok / failed / timeout."""
    args = shlex.split(command)
    if not args:
        return Stats(), "failed"
    iters = option_value(args, ("--iter", "-i"), 100)
    warmup = option_value(args, ("--warmup",), DRIVER_WARMUP)
    holder = None
    if out_dir is None:
        holder = tempfile.TemporaryDirectory()
        cmd_dir = Path(holder.name)
    else:
        cmd_dir = out_dir / f"command_{number}"
        cmd_dir.mkdir(parents=True, exist_ok=True)
    try:
        full = (["rocprofv3", "--output-format", "csv", "--output-directory",
                 str(cmd_dir)] + rocprof_args + ["--", driver] + args)
        if verbose:
            print(f">>> {shlex.join(full)}\n")
        proc = subprocess.run(full, capture_output=True, text=True,
                              timeout=timeout, env=env)
        if verbose and proc.stdout:
            print(proc.stdout)
        if proc.returncode != 0:
            print(f">>> exit code {proc.returncode}\n{proc.stderr[-2000:]}")
            return Stats(), "failed"
        stats = iteration_stats(kernel_durations_us(cmd_dir), iters, warmup)
        if stats.mean == NA:
            print(">>> no kernel dispatches in the trace")
            return stats, "failed"
        print(f">>> Stats: min={stats.min:.2f}(us), max={stats.max:.2f}(us), "
              f"mean={stats.mean:.2f}(us), iter={stats.iter}, "
              f"dispatch_count={stats.dispatch_count}")
        return stats, "ok"
    except subprocess.TimeoutExpired:
        print(f">>> timed out after {timeout} s")
        return Stats(), "timeout"
    except (OSError, RuntimeError, ValueError) as e:
        print(f">>> {e}")
        return Stats(), "failed"
    finally:
        if holder is not None:
            holder.cleanup()


def parser() -> argparse.ArgumentParser:
    here = Path(__file__).resolve().parent
    p = argparse.ArgumentParser(description=__doc__,
                                formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--commands-file", "-f", required=True,
                   help="benchmark commands, one per line")
    p.add_argument("--csv", "-o", default="benchmark_results.csv",
                   help="result table (default: benchmark_results.csv)")
    p.add_argument("--output-dir", "-d", default=None,
                   help="keep the profiler's output here (default: temporary "
                        "directories, removed after each command)")
    p.add_argument("--driver", "-D", default=str(here / "bin" / "driver"),
                   help="benchmark driver binary")
    p.add_argument("--rocprof-args", "-r", default="--kernel-trace",
                   help="trace selection passed to rocprofv3 (default: --kernel-trace)")
    p.add_argument("--verbose", "-v", action="store_true")
    p.add_argument("--timeout", "-t", type=int, default=60,
                   help="seconds per command (default 60, -1: none)")
    p.add_argument("--knob", action="append", default=[], metavar="NAME=VALUE",
                   help="set FUSILLI_HIP_<NAME>=VALUE for the driver (repeatable)")
    return p


def main(argv=None) -> int:
    a = parser().parse_args(argv)
    path = Path(a.commands_file)
    if not path.exists():
        print(f"Error: commands file not found: {path}")
        return 1
    commands = [s for s in (line.strip() for line in open(path))
                if s and not s.startswith("#")]
    if not commands:
        print("Error: no commands found in file")
        return 1
    print(f"Found {len(commands)} commands")
    out_dir = None
    if a.output_dir is not None:
        out_dir = Path(a.output_dir)
        out_dir.mkdir(parents=True, exist_ok=True)
    env = os.environ.copy()
    for kv in a.knob:
        name, _, value = kv.partition("=")
        env["FUSILLI_HIP_" + name] = value
    rocprof_args = shlex.split(a.rocprof_args) or ["--kernel-trace"]
    timeout = None if a.timeout == -1 else a.timeout
    counts = {"ok": 0, "failed": 0, "timeout": 0, "skipped": 0}
    with open(a.csv, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["command"] + [f"{m} (us)" if m in ("min", "max", "mean", "stddev")
                                  else m for m in METRICS])
        for n, command in enumerate(commands, 1):
            bar = "=" * 80
            if command.startswith("[SKIP]"):
                print(f"\n{bar}\nSkipping command {n}/{len(commands)}:\n"
                      f"{command[6:].strip()}\n{bar}\n>>> Skipped")
                stats, outcome = Stats(), "skipped"
            else:
                print(f"\n{bar}\nRunning command {n}/{len(commands)}:\n{command}\n{bar}")
                sys.stdout.flush()
                stats, outcome = run_profiled(command, a.driver, out_dir, rocprof_args,
                                              env, a.verbose, n, timeout)
            counts[outcome] += 1
            w.writerow([command] + [f"{v:.2f}" if isinstance(v, float) else str(v)
                                    for v in stats])
            f.flush()
    print(f"\n{'=' * 80}\nSUMMARY\n{'=' * 80}\nTotal commands: {len(commands)}\n"
          f"Successful: {counts['ok']}\nFailed: {counts['failed']}\n"
          f"Timed out: {counts['timeout']}\nSkipped: {counts['skipped']}\n"
          f"Results CSV: {a.csv}")
    return 0 if counts["failed"] + counts["timeout"] == 0 else 1


if __name__ == "__main__":
    sys.exit(main())
