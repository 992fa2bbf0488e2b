"""Runs the C++ restatement of the reference's GPU tests (tests/host_cpp/test_host.cc): the C++
host mirror of the reference's Rust API, through the C ABI, against the oracle."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "host_cpp", "_build", "test_host")


@pytest.mark.gpu
def test_cpp_host_mirror_passes_the_reference_tests():
    assert os.path.exists(BINARY), "build first: python __graft_entry__.py"
    run = subprocess.run([BINARY], capture_output=True, text=True, timeout=120)
    print(run.stdout[-2000:], run.stderr[-2000:])
    assert run.returncode == 0
    assert "all host tests passed" in run.stdout


def test_cpp_host_mirror_is_built():
    # CPU check: the header compiles against the C ABI and links (done by build()).
    assert os.path.exists(BINARY), "build first: python __graft_entry__.py"
