"""bench.py's command line: more than one GPU is refused with a message (every box of this build has one GPU; the
collectives and sharding of a multi-GPU run are not part of it)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "--gpus must be 1" in (r.stdout + r.stderr)
