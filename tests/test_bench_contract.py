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
    for name in ("cfg2", "cfg3", "cfg4", "cfg5", "pipeline", "accumulate", "resident7b", "multi", "ceilings", "--steps", "--warmup", "--gpus"):
        assert name in res.stdout


def test_traffic_literals_are_the_figures_of_the_committed_summaries():
    """bench.py reports `roofline.traffic` from a table of counter measurements; every entry names
    the summary under profiles/ it was taken from, and that summary states the same number of bytes."""
    import importlib.util
    import re
    spec = importlib.util.spec_from_file_location("bench_for_test", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert set(bench.TRAFFIC_SOURCE) == set(bench.MEASURED_TRAFFIC_BYTES)
    for workload, rel in bench.TRAFFIC_SOURCE.items():
        path = os.path.join(ROOT, rel)
        assert os.path.exists(path), rel
        with open(path) as f:
            found = re.findall(r"roofline\.traffic = ([\d,]+) B", f.read())
        assert found, f"{rel} does not state its roofline.traffic figure"
        assert int(found[-1].replace(",", "")) == bench.MEASURED_TRAFFIC_BYTES[workload], (workload, found)
