"""Runs the C++ test of the drop-in header (tests/cpp/api_test.cpp): the
reference's own usage patterns through nv::merlin::HashTable on the GPU."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cpp", "api_test")


@pytest.mark.gpu
def test_cpp_drop_in_header():
    assert os.path.exists(BINARY), "tests/cpp/api_test is not built: run __graft_entry__.build()"
    r = subprocess.run([BINARY], capture_output=True, text=True, timeout=300)
    print(r.stdout[-4000:])
    print(r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-2000:]
    assert "all checks passed" in r.stdout
