"""The torch-free C++ driver of the C ABI (tests/cabi_driver.cpp, built in-tree by ascend-kernel_amd/build.py):
plain HIP allocations + the library's entry points, checked against the CPU oracle inside the driver."""
import os
import subprocess

import pytest

import oracle

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "ascend-kernel_amd", "cabi_driver")


def test_cabi_driver_runs_clean():
    assert os.path.exists(DRIVER), "build it with `python ascend-kernel_amd/build.py`"
    lib = oracle.build()
    print("running", DRIVER, flush=True)
    r = subprocess.run([DRIVER, lib], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "cabi_driver ok" in r.stdout
