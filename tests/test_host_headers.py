"""Host-side arithmetic of the C++ headers that can be checked without a GPU (compiled with g++ here)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_split_walk_integer_bound_equals_float_test(tmp_path):
    exe = tmp_path / "accept_below"
    src = os.path.join(ROOT, "tests", "host_checks", "accept_below.cpp")
    subprocess.run(["g++", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "include"), src, "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "mismatches 0" in out.stdout
