"""The C ABI from a host without Python or torch: tests/cabi_host.cpp links libaicomp_kv.so,
runs one fused append + decode step and checks it itself; the test runs the built program."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def test_cpp_host_program(device):
    exe = os.path.join(HERE, "cabi_host")
    assert os.path.exists(exe), "tests/cabi_host is missing: run `python -m aicomp_amd.build`"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, f"cabi_host failed ({r.returncode}):\n{r.stdout}\n{r.stderr}"
    assert "append bit-exact" in r.stdout
