"""bench.py without a GPU: more than one GPU is refused with one line and exit code 2."""

import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "3", "--warmup", "1"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    assert len(proc.stdout.strip().splitlines()) == 1 and "one GPU" in proc.stdout
