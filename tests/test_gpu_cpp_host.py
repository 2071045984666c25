"""Runs the C++ restatement of the reference's k-quant kernel tests
(tests/cpp/kernel_test.cpp) against the host layer and the C ABI on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "kernel_test")


def test_reference_kernel_tests_through_cpp_host_layer():
    assert os.path.exists(BIN), "tests/cpp/kernel_test is missing: run `make -C tests/cpp` (build() does)"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "16 tests, 0 failed" in r.stdout
