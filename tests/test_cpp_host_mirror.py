"""The C++ host-side mirror (include/tract_rocm.hpp) and its test program, which restates the
reference's unit tests for the in-place cache and the fused op in C++."""
import os
import subprocess

import pytest

from tests.conftest import ROOT

SRC = os.path.join(ROOT, "tests", "cpp", "host_mirror_test.cpp")
BIN = os.path.join(ROOT, "tests", "cpp", "host_mirror_test")


def build_cpp_test():
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), SRC,
                    "-L", os.path.join(ROOT, "tract_amd"), "-ltract_rocm", "-Wl,-rpath,$ORIGIN/../../tract_amd",
                    "-o", BIN], check=True)


def test_cpp_mirror_compiles_and_links():
    build_cpp_test()
    assert os.path.exists(BIN)


@pytest.mark.gpu
def test_cpp_mirror_runs_on_gpu():
    if not os.path.exists(BIN):
        build_cpp_test()
    p = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "all checks passed" in p.stdout
