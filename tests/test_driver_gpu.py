"""Graph-API benchmark driver (fusilli_amd/bench): every command of its
test_commands.txt — the reference's benchmarks/test_commands.txt plus the
benchmark configs — must run, plan to a single fused kernel and print one CSV
row with the `iter` and `dispatch_count` columns the reference's runner checks
(benchmarks/test_benchmark_runner.sh:22-43)."""
import os
import shlex
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "fusilli_amd", "bench", "bin", "driver")
COMMANDS = os.path.join(ROOT, "fusilli_amd", "bench", "test_commands.txt")


def commands():
    out = []
    for line in open(COMMANDS):
        line = line.strip()
        if line and not line.startswith("#") and not line.startswith("[SKIP]"):
            out.append(line)
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("cmd", commands())
def test_driver_command(cmd):
    assert os.path.exists(DRIVER), \
        f"{DRIVER} missing: run `python -c 'import __graft_entry__ as g; g.build()'`"
    proc = subprocess.run([DRIVER] + shlex.split(cmd), capture_output=True,
                          text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.strip().splitlines()
    header, row = lines[-2].split(","), lines[-1].split(",")
    assert header[:4] == ["name", "iter", "dispatch_count", "avg_us"]
    rec = dict(zip(header, row))
    want_iter = shlex.split(cmd)[shlex.split(cmd).index("--iter") + 1]
    assert rec["iter"] == want_iter
    assert rec["dispatch_count"] == "1"  # producer + pointwise chain fused
    assert float(rec["avg_us"]) > 0


def test_driver_commands_file_has_every_subcommand():
    subs = {shlex.split(c)[[i for i, t in enumerate(shlex.split(c))
                            if not t.startswith("-") and not t.isdigit()][0]]
            for c in commands()}
    assert {"conv", "matmul", "sdpa", "layernorm", "rmsnorm"} <= subs
