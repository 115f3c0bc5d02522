"""The benchmark script's command line, as far as it can be exercised without a GPU."""
from __future__ import annotations

import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def run(*args, env=None):
    return subprocess.run([sys.executable, BENCH, *args], capture_output=True, text=True,
                          timeout=300, env=env)


def test_help_prints_every_option():
    r = run("--help")
    assert r.returncode == 0, r.stderr
    for flag in ("--gpus", "--steps", "--warmup", "--workload", "--wgrad-group", "--two-streams",
                 "--graph", "--kernel-table", "--mfma-ceiling", "--after-loop"):
        assert flag in r.stdout, flag


@pytest.mark.parametrize("n", ["2", "8"])
def test_more_than_one_gpu_is_refused_with_a_message(n):
    r = run("--gpus", n)
    assert r.returncode != 0
    assert "one GPU" in r.stderr + r.stdout
    assert not r.stdout.strip().startswith("{")     # no result line


def test_a_multi_rank_launch_is_refused_too():
    env = dict(os.environ, WORLD_SIZE="2", RANK="0", LOCAL_RANK="0",
               MASTER_ADDR="127.0.0.1", MASTER_PORT="29512")
    r = run("--gpus", "1", env=env)
    assert r.returncode != 0
    assert not r.stdout.strip().startswith("{")


def test_unknown_workload_is_an_error():
    r = run("--workload", "cfg9")
    assert r.returncode != 0
    assert "cfg9" in r.stderr


def test_without_a_gpu_the_run_fails_loudly():
    """No CPU path stands in for the HIP library: on a host without a device the script ends
    with an error and prints no result line."""
    if os.path.exists("/dev/kfd"):      # asked of the file system: no HIP call in this process
        pytest.skip("a GPU may be visible")
    r = run("--no-cpu-baseline", "--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "GPU" in r.stderr
    assert not r.stdout.strip().startswith("{")
