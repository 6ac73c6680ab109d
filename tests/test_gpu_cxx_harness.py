"""Runs the C++ harness (tests/cxx/km_harness.cc) that drives the kernel manager through the
header-only C++ class with the reference's member names and checks it against the oracle."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "cxx", "km_harness")


@pytest.mark.gpu
def test_cxx_harness_passes():
    assert os.path.exists(BINARY), "build it with __graft_entry__.build()"
    r = subprocess.run([BINARY], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and r.stdout.strip().endswith("PASS"), r.stdout + r.stderr
