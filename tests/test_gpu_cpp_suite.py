"""Runs the C++ rendition of the reference crate's test suite
(tests/cpp/test_symmetric.cpp, built by cubek_amd/csrc/Makefile) on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BINARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "test_symmetric")


def test_reference_suite_through_cpp_host_layer():
    assert os.path.exists(BINARY), "tests/cpp/test_symmetric is not built (make -C cubek_amd/csrc)"
    proc = subprocess.run([BINARY], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(proc.stdout)
    lines = [l for l in proc.stdout.splitlines() if l.startswith(("PASS", "FAIL"))]
    assert proc.returncode == 0, proc.stdout
    assert len([l for l in lines if l.startswith("PASS")]) == 24 + 4 + 2 + 1 and not [l for l in lines if l.startswith("FAIL")]
