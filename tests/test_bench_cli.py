"""bench.py's command line, as far as it can be checked without a GPU: this executor path runs on one GPU, and asking
for more is refused with a message before anything touches a device."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 2
    assert "ONE GPU" in out.stderr and out.stdout.strip() == ""


def test_help_lists_the_profiling_modes():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0
    for flag in ("--matmul-only", "--chain-only", "--block-only", "--attention-only", "--in-order-only", "--no-cpu", "--no-per-op"):
        assert flag in out.stdout, flag
