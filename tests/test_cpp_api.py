"""Runs the C++ graph-API test binaries (tests/cpp).  The host binary needs no
GPU; the device binary runs the reference samples' known answers end to end on
Backend::AMDGPU."""
import os
import subprocess
import tempfile

import pytest

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "bin")


def _run(name, timeout):
    path = os.path.join(BIN, name)
    assert os.path.exists(path), \
        f"{path} missing: run `python -c 'import __graft_entry__ as g; g.build()'`"
    # the graphs' cache files go to a directory of this run
    with tempfile.TemporaryDirectory(prefix="fusilli_cache_") as cache:
        env = dict(os.environ, FUSILLI_CACHE_DIR=cache)
        proc = subprocess.run([path], capture_output=True, text=True,
                              timeout=timeout, env=env)
        left = [os.path.join(d, f) for d, _, fs in os.walk(cache) for f in fs]
    # every test compiles with remove = true or cleans up after itself
    # (reference tests/test_cache_empty.sh)
    assert not left, f"{name} left cache files behind: {left[:5]}"
    tail = "\n".join(proc.stdout.splitlines()[-60:])
    assert proc.returncode == 0, f"{name} failed:\n{tail}\n{proc.stderr[-2000:]}"
    assert "0 failed checks" in proc.stdout, tail
    return proc.stdout


def test_cpp_host_api():
    out = _run("test_host_api", 120)
    assert "19 cases" in out or "cases, 0 failed" in out


def test_cpp_node_validation():
    """The reference's node / attribute validation expectations (codes, exact
    messages, order of checks): tests/cpp/test_node_validation.cpp."""
    out = _run("test_node_validation", 120)
    assert "cases, 0 failed" in out


@pytest.mark.gpu
def test_cpp_device_api():
    _run("test_device_api", 300)
