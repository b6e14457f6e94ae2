"""The public C++ headers (include/ark/*.hpp) as a user of the reference would use them: a
program that includes <ark/ark.hpp>, links -larkmi and goes through ark::Model,
ark::Planner rules and ark::DefaultExecutor (tests/cpp/drop_in_executor.cpp, built by
tests/cpp/Makefile ahead of time).  The program compares a matmul + add with a host loop
bit for bit and exits non-zero on any mismatch."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def test_cpp_program_against_public_headers():
    exe = os.path.join(HERE, "cpp", "drop_in_executor")
    assert os.path.exists(exe), "build it first: make -C tests/cpp"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "drop_in_executor: OK" in r.stdout
