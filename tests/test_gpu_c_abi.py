"""The C ABI from plain C: ``tests/abi_driver.c`` (C99 + the HIP runtime, no Python, no PyTorch) builds a plan,
runs the fused step, the allocation-free entry point, an overflow case, a cast copy and two error paths, and
checks every result against values it computes on the host itself.  ``rannc_amd/build.py`` compiles it."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "tests", "abi_driver")


@pytest.mark.gpu
def test_c_driver_runs_the_abi_without_python():
    if not os.path.exists(DRIVER):
        pytest.fail("tests/abi_driver is not built: run python rannc_amd/build.py")
    proc = subprocess.run([DRIVER], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert proc.returncode == 0 and "abi_driver: OK" in proc.stdout, proc.stdout
