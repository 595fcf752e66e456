"""Runs the native C++ tests of the host class tokspur::HipGraph (tests/native/*.cpp, built by
__graft_entry__.build() into tests/native/bin/) on the GPU and reports their output."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "bin")


@pytest.mark.parametrize("name", ["test_hip_graph"])
def test_native(name):
    path = os.path.join(BIN, name)
    assert os.path.exists(path), f"{path} is not built: run __graft_entry__.build()"
    proc = subprocess.run([path], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout[-4000:]
