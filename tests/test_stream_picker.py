"""Which stream a launch goes to when independent launches of a batch may overlap (deepx_amd/executor/stream_picker.hpp)
is plain host C++: compiled with g++ and exercised here without a GPU — 600 random programs replayed in a
happens-before model, in which every read-after-write, write-after-read and write-after-write pair must be ordered."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_stream_picker(tmp_path):
    exe = str(tmp_path / "stream_picker_check")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-Wall", "-I", os.path.join(ROOT, "deepx_amd", "executor"),
                           os.path.join(ROOT, "tests", "stream_picker_check.cpp"), "-o", exe])
    out = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stdout + out.stderr
