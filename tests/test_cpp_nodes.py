"""Runs the C++ test driver of the drop-in node classes
(tests/cpp/test_nodes.cpp, built by coalsack_amd/host/Makefile)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "coalsack_amd", "host", "build", "test_nodes")


def _run(mode):
    assert os.path.exists(BIN), f"{BIN} is missing: run __graft_entry__.build()"
    p = subprocess.run([BIN, mode], capture_output=True, text=True, timeout=120)
    print(p.stdout)
    print(p.stderr)
    assert p.returncode == 0, p.stdout[-2000:]
    assert " 0 failed" in p.stdout


def test_node_argument_and_error_paths():
    _run("--cpu")


@pytest.mark.gpu
def test_node_numerics_on_gpu():
    _run("--gpu")
