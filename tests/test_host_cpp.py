"""Runs the C++ tests of the host mirror (include/wrq.hpp, tests/cpp/test_host.cpp)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_host")


def build_host_tests():
    subprocess.run(
        ["/opt/rocm/bin/hipcc", "-std=c++17", "-O1", "-o", BIN, os.path.join(ROOT, "tests", "cpp", "test_host.cpp"),
         "-L" + os.path.join(ROOT, "web-rwkv_amd"), "-lwrq_hip", "-Wl,-rpath,$ORIGIN/../../web-rwkv_amd"],
        check=True, capture_output=True)


def run(args):
    if not os.path.exists(BIN):
        build_host_tests()
    r = subprocess.run([BIN] + args, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "host tests ok" in r.stdout


def test_host_mirror_schedule_and_errors():
    # token schedule KATs of src/runtime/infer/rnn.rs:362-569 and op-build shape errors; no device needed
    run(["--cpu"])


@pytest.mark.gpu
def test_host_mirror_drives_the_gpu():
    print("case: C++ host mirror, one v6-shaped layer through Queue::submit", flush=True)
    run([])
