"""bench.py's command line: what can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_unknown_leg_is_refused():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--only", "nothing"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0 and "invalid choice" in proc.stderr
