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
# every add_fusilli_benchmark command of the reference's
# benchmarks/CMakeLists.txt:49-392, extracted as data
REFERENCE_COMMANDS = os.path.join(ROOT, "fusilli_amd", "bench",
                                  "reference_commands.txt")


def commands(path=COMMANDS):
    out = []
    for line in open(path):
        line = line.strip()
        if line and not line.startswith("#") and not line.startswith("[SKIP]"):
            out.append(line)
    return out


def run_verified(cmd):
    """Runs one driver command with --verify: besides timing, the driver then
    compares every element of every output with the closed form its constant
    fills imply (convolution: taps inside the image x channels of a group;
    matmul: K; attention over constant tensors: V; the norms' constant-row
    answers) and fails on a mismatch.  Returns the CSV row as a dict."""
    proc = subprocess.run([DRIVER, "--verify"] + shlex.split(cmd), capture_output=True,
                          text=True, timeout=180)
    assert proc.returncode == 0, (proc.stdout[-1500:] + proc.stderr[-2000:])
    lines = proc.stdout.strip().splitlines()
    checks = [ln.split(",") for ln in lines if ln.startswith("verify,")]
    assert checks, "no output was verified"
    for _, name, elements, mismatches, _worst in checks:
        assert int(elements) > 0 and int(mismatches) == 0, (name, mismatches)
    timing = [ln for ln in lines if not ln.startswith("verify,")]
    header, row = timing[-2].split(","), timing[-1].split(",")
    assert header[:4] == ["name", "iter", "dispatch_count", "avg_us"]
    return dict(zip(header, row))


@pytest.mark.gpu
@pytest.mark.parametrize("cmd", commands())
def test_driver_command(cmd):
    assert os.path.exists(DRIVER), \
        f"{DRIVER} missing: run `python -c 'import __graft_entry__ as g; g.build()'`"
    rec = run_verified(cmd)
    want_iter = shlex.split(cmd)[shlex.split(cmd).index("--iter") + 1]
    assert rec["iter"] == want_iter
    assert rec["dispatch_count"] == "1"  # producer + pointwise chain fused
    assert float(rec["avg_us"]) > 0


@pytest.mark.gpu
@pytest.mark.parametrize("cmd", commands(REFERENCE_COMMANDS))
def test_driver_runs_the_reference_benchmark_commands(cmd):
    # 2-D and 3-D convolutions in every direction and layout, layer norms of
    # rank 2 to 4, (batched, transposed, mixed-type) matmuls, attention with
    # mask / GQA / explicit scale: each must run unchanged and print its row.
    rec = run_verified(cmd)
    assert rec["iter"] == "10"
    # gradients with --bias add the bias-gradient reduction as a second step
    steps = 2 if ("--bias" in cmd and (" -F 2 " in cmd or " -F 4 " in cmd)) else 1
    assert int(rec["dispatch_count"]) == steps
    assert float(rec["avg_us"]) > 0


@pytest.mark.parametrize("bad", [
    "conv -F 1 -n 1 -c 8 -H 8 -W 8 -k 8 -y 3 -x 3 -p 1 -q 1 -u 1 -v 1 -l 1 -j 1 "
    "--in_layout NHWC --out_layout NHWC --fil_layout NHWC --spatial_dim 2 --nonsense 3",
    "conv -F 1 -n 1 -c 8 -H 8 -W 8 -k 8 -y 3 -x 3 -p 1 -q 1 -u 1 -v 1 -l 1 -j 1 "
    "--in_layout NDHWC --out_layout NDHWC --fil_layout NDHWC --spatial_dim 2",
    "conv -F 1 -n 1 -c 8 -H 8 -W 8 -k 8 -y 3 -x 3 -p 1 -q 1 -u 1 -v 1 -l 1 -j 1 "
    "--in_layout NDHWC --out_layout NDHWC --fil_layout NDHWC --spatial_dim 3",
    "matmul -M 16 -N 32 -K 64 --a_type f32 --b_type f32 --out_type f32 --transC",
    "sdpa -B 1 --heads_q 8 --heads_kv 8 --seq_q 64 --seq_kv 64 -d 64 -t f16 --causal --mask",
    "layernorm -X 2x3x128 -F 1 -t f32 --layout NCHW",
])
def test_driver_rejects_what_it_does_not_implement(bad):
    # unknown flags, layouts of the wrong rank, 3-D without its depth flags:
    # an error before any device is touched, never a number for another problem
    proc = subprocess.run([DRIVER] + shlex.split(bad), capture_output=True,
                          text=True, timeout=60)
    assert proc.returncode != 0
    assert "driver:" in proc.stderr


def test_driver_commands_file_has_every_subcommand():
    subs = {shlex.split(c)[[i for i, t in enumerate(shlex.split(c))
                            if not t.startswith("-") and not t.isdigit()][0]]
            for c in commands()}
    assert {"conv", "matmul", "sdpa", "layernorm", "rmsnorm"} <= subs
