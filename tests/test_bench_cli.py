"""The benchmark's command line, without a GPU: more than one GPU is refused with a message, before anything is imported
that would need one."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr + r.stdout
    assert not r.stdout.strip().startswith("{")  # no result line
