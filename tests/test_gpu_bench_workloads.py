"""Every workload of bench.py that finishes in seconds runs and prints its one JSON line (the large
ones -- the default line with its sub-records, cfg5, resident7b -- are what the round's bench runs
are for). Small shapes where the workload takes them; nothing is asserted about speed."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
QUIET = ["--no-cpu-baseline", "--no-offload-record", "--no-side-records"]


@pytest.mark.parametrize("argv,keys", [
    (["--workload", "cfg3", "--steps", "3", "--warmup", "1", *QUIET], ["roofline", "stats_pass", "guarded_step"]),
    (["--workload", "accumulate", "--steps", "3", "--warmup", "1", *QUIET], ["roofline", "variants"]),
    (["--workload", "multi", "--steps", "3", "--warmup", "1", *QUIET], ["roofline", "variants"]),
    (["--workload", "pipeline", "--resident", "--layers", "2", "--micro-batches", "4", "--steps", "2", "--warmup", "1"], ["roofline"]),
    (["--workload", "pipeline", "--resident", "--layers", "2", "--micro-batches", "4", "--layer-groups", "--step-stream", "on",
      "--steps", "2", "--warmup", "1"], ["roofline"]),
    (["--workload", "pipeline", "--layers", "2", "--micro-batches", "4", "--steps", "2", "--warmup", "1"], ["roofline"]),
    (["--workload", "pipeline", "--layers", "2", "--micro-batches", "4", "--alpha", "0.25", "--steps", "2", "--warmup", "1"], ["roofline"]),
])
def test_workload_runs(cuda, argv, keys):
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *argv], capture_output=True, text=True, timeout=170)
    assert run.returncode == 0, run.stdout[-1500:] + run.stderr[-1500:]
    line = json.loads(run.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "n_gpus", "ms_per_step", *keys):
        assert key in line, (key, sorted(line))
    assert line["n_gpus"] == 1 and line["value"] > 0
