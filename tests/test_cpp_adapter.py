"""The C++ adapter above the C-ABI (dynet_amd/adapter/dynet_hip_adapter.h) driven by tests/cpp/test_adapter.cpp,
which replays the reference's node tests (tests/test-rnn.cc, tests/test-nodes.cc) in C++."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_adapter")


def _binary():
    if not os.path.exists(BIN):  # built by __graft_entry__.build(); fall back to building it here
        subprocess.run(["make", "-C", os.path.dirname(BIN)], check=True)
    return BIN


def test_adapter_links_and_reports_a_missing_device_as_cuda_exception():
    r = subprocess.run([_binary(), "--no-gpu"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr


@pytest.mark.gpu
def test_reference_node_tests_through_the_cpp_adapter():
    r = subprocess.run([_binary()], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "0 failed" in r.stdout
