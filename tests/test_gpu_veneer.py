"""Runs the C++ host veneer's own test program (tests/cpp/veneer_test.cpp): the
dlf-style DevTensor front-ends over gpgpu::dnn over the C ABI, against the
reference's literal vectors."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "veneer_test.bin")


def test_cpp_veneer_program():
    assert os.path.exists(BIN), "run __graft_entry__.build() first"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "0 failed" in r.stdout
