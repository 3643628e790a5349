"""Runs the C++ class-shell program (tests/cpp/test_shells.cpp): cagra::CagraIndex, cagra::CagraIndexOpt and
cagra::DeviceBufferVMM with the reference's method names over the C ABI."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "_bin", "test_shells")


def _need_bin():
    if not os.path.exists(BIN):
        pytest.fail(f"{BIN} is not built: run __graft_entry__.build() or `make -C tests/cpp`")


def test_shells_fail_loudly_without_gpu():
    _need_bin()
    r = subprocess.run([BIN, "--no-gpu"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "PASSED" in r.stdout or "SKIPPED" in r.stdout


@pytest.mark.gpu
def test_shells_on_gpu():
    _need_bin()
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0 and "PASSED" in r.stdout, r.stdout + r.stderr
