"""bench.py's contract where no GPU is needed: more than one GPU is refused with one line and exit code 2."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_one_line():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "3", "--warmup", "1"],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode == 2
    lines = [line for line in proc.stdout.split("\n") if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]
