"""The bookkeeping of the device-block pool (deepx_amd/csrc/block_pool.hpp) is plain host C++ over two function
pointers: compiled with g++ and run here against a fake driver with a byte budget — size classes, reuse, the cap,
refusal of foreign and repeated pointers, giving everything back when the driver runs out."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_block_pool(tmp_path):
    exe = str(tmp_path / "block_pool_check")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-Wall", "-I", os.path.join(ROOT, "deepx_amd", "csrc"),
                           os.path.join(ROOT, "tests", "block_pool_check.cpp"), "-o", exe])
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stdout + out.stderr
