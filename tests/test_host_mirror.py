"""The C++ host mirror (include/llmp_hip.hpp) through its own test program
(tests/host/mirror_test.cc, built by __graft_entry__.build()): the reference's launch
interfaces by name over the C ABI, checked from C++ the way the reference's unit tests do."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
PROGRAM = os.path.join(HERE, "host", "mirror_test")


def run(mode):
    if not os.path.exists(PROGRAM):
        subprocess.run(["make", "-C", os.path.join(HERE, "host")], check=True, capture_output=True)
    done = subprocess.run([PROGRAM, mode], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stdout + done.stderr
    return done.stdout


def test_refusals_and_layout_arithmetic_from_cpp():
    assert "host checks: 0 failure(s)" in run("host")


@pytest.mark.gpu
def test_products_from_cpp_match_the_oracle():
    out = run("device")
    assert "device checks: 0 failure(s)" in out, out
