"""Host-side contract of the C++ layer (backpack_amd/csrc/host): a Q6_K weight view must carry the 16 readable
bytes behind its last row that the kernels' 16-byte fetches need (include/bpk_kquant.h, bpk_kq_matmul), as
uploadKQWeight (the counterpart of runtime/model_runner.cpp:958-963) allocates them.  The checks touch no device."""
import os
import subprocess

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "kernel_test")


def test_weight_view_checks_without_a_device():
    assert os.path.exists(BIN), "tests/cpp/kernel_test is missing: run `make -C tests/cpp` (build() does)"
    r = subprocess.run([BIN, "--host-only"], capture_output=True, text=True, timeout=60)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "0 host-only checks failed" in r.stdout
    assert r.stdout.count("PASS") == 9
