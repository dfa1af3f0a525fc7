"""bench.py's contract where no GPU is needed: more than one GPU is refused in one line with exit code 2."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_in_one_line():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                         capture_output=True, text=True, timeout=120)
    assert run.returncode == 2
    lines = [l for l in run.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]
