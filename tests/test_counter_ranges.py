"""The bookkeeping behind counters that recorded launches own (deepx_amd/csrc/counter_ranges.hpp) is plain
host C++: compiled with g++ and exercised here without a GPU — a server that records and drops graphs for
ever never runs out, failed captures return at once, nothing is handed out twice."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_counter_ranges(tmp_path):
    exe = str(tmp_path / "counter_ranges_check")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-Wall", "-I", os.path.join(ROOT, "deepx_amd", "csrc"),
                           os.path.join(ROOT, "tests", "counter_ranges_check.cpp"), "-o", exe])
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stdout + out.stderr
