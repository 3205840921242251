"""bench.py's command line, as far as it can be checked without a GPU."""

import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def test_more_than_one_gpu_is_refused_with_a_message():
    """The path has no multi-GPU component: `--gpus N` with N above 1 exits before touching a
    device, non-zero, and says why."""
    res = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert res.returncode != 0
    assert "one GPU" in res.stderr and "--gpus 2" in res.stderr
    assert res.stdout.strip() == ""  # no JSON line that a harness could mistake for a measurement
