"""Runs the C++ host-side test program (tests/cpp/sparse_conv_hip_test.cc):
detect pass -> SparseConvOp -> registered TARGET(kHIP) kernel -> Launch."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "sparse_conv_hip_test")


def _run(mode):
    assert os.path.exists(BIN), "build the host test first: python -c 'import __graft_entry__ as g; g.build()'"
    res = subprocess.run([BIN, mode], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(res.stdout)
    assert res.returncode == 0, res.stdout[-4000:]
    assert "0 failure(s)" in res.stdout


def test_registry_op_and_pass_on_host():
    _run("--cpu")


@pytest.mark.gpu
def test_whole_op_path_on_device():
    _run("--gpu")
