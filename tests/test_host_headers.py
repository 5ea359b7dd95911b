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


def _build(tmp_path, source, name, extra=()):
    exe = tmp_path / name
    subprocess.run(["g++", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "include"), *extra,
                    os.path.join(ROOT, "tests", "host_checks", source), "-o", str(exe)], check=True)
    return exe


def test_utils_header_matches_the_oracle_and_closed_forms(tmp_path, oracle):
    """superkmeans/pdx/utils.h (TicToc, MakeBlobs, GenerateRandomVectors, brute-force checkers: what the reference's
    examples and tests include next to the clustering classes).  MakeBlobs on one thread equals the oracle's
    restatement of pdx/utils.h:74-123 bit for bit; the rest is checked against hand-computed values."""
    import numpy as np

    # same code generation options as the oracle (oracle/Makefile): libstdc++'s normal_distribution is inlined, and
    # whether its scale-and-shift is fused with the addition of the centre depends on them
    exe = _build(tmp_path, "utils_header.cpp", "utils_header", extra=("-O3", "-march=x86-64-v3"))
    lines = dict(l.split(" ", 1) for l in subprocess.run([str(exe)], capture_output=True, text=True, check=True)
                 .stdout.strip().splitlines())
    got = np.array(lines["blobs"].split(), dtype=np.float32).reshape(50, 7)
    assert np.array_equal(got, oracle.make_blobs(50, 7, 5, False, 0.25, 5.0, 42))
    assert float(lines["unit_norm_error"]) < 1e-5
    lo, hi = map(float, lines["uniform_range"].split())
    assert -2.0 <= lo < -1.5 and 2.5 < hi < 3.0
    assert lines["nn"].split() == ["1", "2", "0.0100", "1.0000"]
    assert lines["knn"].split() == ["1", "0", "2", "1"]
    assert lines["nearest_centroid"] == "2"
    assert lines["rounding"].split() == ["128", "64", "1", "0"]
    assert lines["below"] == "30"
    assert lines["timer_ok"] == "1"


def test_shuffled_prefix_equals_std_shuffle(tmp_path):
    """GenerateCentroids keeps the first k entries of std::shuffle over all n indices (reference superkmeans.h:1100-1120).
    ShuffledPrefix derives them from the draws alone for large n; it must give the entries, and leave the generator in
    the state, that shuffling the whole array gives: n on both sides of its size switch and of libstdc++'s own switch
    at 65,536, k = 1, 5, n/3 and n, two seeds."""
    exe = _build(tmp_path, "shuffled_prefix.cpp", "shuffled_prefix")
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "mismatches 0" in out.stdout
    assert "equal 1" in out.stdout


def test_reference_examples_compile_against_these_headers():
    """The reference's own example programs use nothing but the public headers: they must pass a syntax check
    against include/ unchanged.  Skipped where the reference checkout is absent."""
    import glob

    import pytest

    examples = sorted(glob.glob("/root/reference/examples/*.cpp"))
    if not examples:
        pytest.skip("reference checkout not present")
    for src in examples:
        out = subprocess.run(["g++", "-fsyntax-only", "-std=c++17", "-fopenmp", "-I", os.path.join(ROOT, "include"), src],
                             capture_output=True, text=True)
        assert out.returncode == 0, f"{src}:\n{out.stderr[-2000:]}"
