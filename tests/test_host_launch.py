"""The HIP device-execution provider and launch context (include/llmp_hip_launch.h and .hpp) through their own test
program (tests/host/launch_test.cc, built by __graft_entry__.build()): the reference's DeviceExecution and
LaunchContext interfaces by name, driven from C++ as the reference's executor drives them."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
PROGRAM = os.path.join(HERE, "host", "launch_test")


def run(mode):
    if not os.path.exists(PROGRAM):
        subprocess.run(["make", "-C", os.path.join(HERE, "host"), "launch_test"], check=True, capture_output=True)
    done = subprocess.run([PROGRAM, mode], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stdout + done.stderr
    return done.stdout


def test_refusals_without_a_device():
    assert "host checks: 0 failure(s)" in run("host")


@pytest.mark.gpu
def test_runs_captures_lanes_and_fences_on_the_device():
    out = run("device")
    assert "device checks: 0 failure(s)" in out, out
