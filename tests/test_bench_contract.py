"""bench.py's contract for more than one GPU: one line that says so, exit code 2 (no GPU needed)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    assert len(proc.stdout.strip().splitlines()) == 1 and "one GPU" in proc.stdout


import json

import pytest


@pytest.mark.gpu
def test_bench_serving_workload_prints_its_line():
    """``--workload serve3b`` in small (one layer of the 28, five requests): the whole engine runs the requests to
    their end and one JSON line says what was measured."""
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "serve3b", "--layers", "1",
                           "--requests", "5"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    assert d["n_gpus"] == 1 and d["unit"] == "tokens/s" and d["value"] > 0 and d["dtype"] == "bf16"
    assert d["config"]["layers"] == 1 and d["config"]["layers_full"] == 28 and d["config"]["requests"] == 5
    assert d["generated_tokens"] == 5 * 256 and d["prompt_tokens"] >= 5 * 128 and d["steps"] >= 256
    assert len(d["config"]) <= 20 and all(not isinstance(v, (dict, list)) for v in d["config"].values())
