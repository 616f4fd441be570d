"""Runs csrc/engine_path_test (tests/cpp/test_engine_path.cpp, built by the package's build
step): the C++ drop-in classes used the way the engine uses its ForwardPipe, compared bit for
bit with the C-ABI path."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "leela-zero_amd", "csrc", "engine_path_test")
pytestmark = pytest.mark.gpu


def test_engine_path_binary():
    print("case: engine_path_test", flush=True)
    assert os.path.exists(EXE), "run __graft_entry__.build() first"
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "engine path ok" in r.stdout
