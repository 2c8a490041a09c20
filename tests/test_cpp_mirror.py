"""The reference's unit tests for this path, re-expressed in C++ against the host mirror
include/allpaka_backend.hpp (tests/cpp/test_mirror.cpp), run on the GPU through the C ABI."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_mirror")


def test_cpp_mirror_builds_and_declines_without_a_gpu():
    """CPU-side: the header compiles against the C ABI and links the library; with the GPU path
    disabled by ALLPAKA_NO_GPU (capability.rs:58-61) the backend declines instead of failing."""
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "tests", "cpp")])
    env = dict(os.environ, ALLPAKA_NO_GPU="1")
    r = subprocess.run([BIN], env=env, capture_output=True, text=True, timeout=60)
    assert r.returncode == 77 and "ALLPAKA_NO_GPU" in r.stdout


@pytest.mark.gpu
def test_cpp_mirror_reference_unit_tests():
    assert os.path.exists(BIN), "tests/cpp/test_mirror is not built (python -c 'import __graft_entry__ as g; g.build()')"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(r.stdout[-3000:])
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-1000:]
    assert "0 failure(s)" in r.stdout
