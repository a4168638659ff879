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
