"""The HIP device-memory provider (include/llmp_hip_memory.h and .hpp) through its own test program
(tests/host/memory_test.cc, built by __graft_entry__.build()): the reference's DeviceMemory interface by name. The rules
that every implementation of it shares run on the CPU over primitives that fail on request; the device checks map real
backing and move bytes through it."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
PROGRAM = os.path.join(HERE, "host", "memory_test")


def run(mode):
    if not os.path.exists(PROGRAM):
        subprocess.run(["make", "-C", os.path.join(HERE, "host"), "memory_test"], check=True, capture_output=True)
    done = subprocess.run([PROGRAM, mode], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stdout + done.stderr
    return done.stdout


def test_the_shared_rules_over_primitives_that_fail_on_request():
    assert "rules checks: 0 failure(s)" in run("rules")


def test_refusals_without_a_device():
    assert "host checks: 0 failure(s)" in run("host")


@pytest.mark.gpu
@pytest.mark.skip(reason="the one run of the HIP virtual memory primitives on an MI355X (two mappings, access granted, host "
                         "copies through them) left the GPU faulted and its cause has not been shown: llmp_hip_memory_open "
                         "refuses in the default build, and this case stays off the GPU until a cause is shown")
def test_reservations_backing_and_mappings_on_the_device():
    out = run("device")
    assert "device checks: 0 failure(s)" in out, out
