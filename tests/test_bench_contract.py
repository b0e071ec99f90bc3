"""bench.py's command-line contract that needs no GPU."""

import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    """One GPU stands in for the group: `--gpus N` with N > 1 exits and says why."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stdout + r.stderr) and "--gpus" in (r.stdout + r.stderr), r.stdout + r.stderr
