"""The parts of bench.py's contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*argv):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *argv], capture_output=True, text=True, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    res = _run("--gpus", "2")
    assert res.returncode == 2
    assert "--gpus must be 1" in res.stderr and not res.stdout.strip()


def test_help_names_every_workload():
    res = _run("--help")
    assert res.returncode == 0
    for name in ("cfg2", "cfg3", "cfg4", "cfg5", "pipeline", "accumulate", "resident7b", "--steps", "--warmup", "--gpus"):
        assert name in res.stdout
