"""Runs the C++ host-layer test program (tests/cpp/host_api_tests.cpp), which
mirrors the reference's xUnit suites through the C++ counterpart of the C#
API.  The binary is built by ``python -m ilgpu_amd.build``."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "cpp", "host_api_tests")


def run(*args):
    assert os.path.exists(BINARY), "build it with `python -m ilgpu_amd.build`"
    proc = subprocess.run([BINARY, *args], capture_output=True, text=True,
                          timeout=300)
    print(proc.stdout[-4000:])
    print(proc.stderr[-2000:])
    return proc


def test_temp_view_manager_rules_on_host():
    proc = run("--host")
    assert proc.returncode == 0
    assert "0 failed checks" in proc.stdout


@pytest.mark.gpu
def test_reference_suites_through_the_cpp_host_layer():
    proc = run()
    assert proc.returncode == 0, proc.stdout[-2000:]
    assert "0 failed checks" in proc.stdout
