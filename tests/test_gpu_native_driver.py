"""A C++ host program (tests/native/abi_driver.cpp) drives the library through the C ABI with
hipMalloc'd buffers -- no torch, no Python in the process -- and checks every hot-path entry point
against float64 evaluations of the reference's formulas."""

import subprocess

import pytest

pytestmark = pytest.mark.gpu


def test_cpp_host_program_passes_its_checks(dev):
    from tests.native.build import DRIVER, build_driver

    if not DRIVER.exists():  # normally prebuilt with the library; build only if absent
        build_driver(verbose=False)
    proc = subprocess.run([str(DRIVER)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout[-2000:]
    assert "all checks passed" in proc.stdout
    for part in ("token log-prob + entropy", "sde step + log-prob", "gaussian kl + mask", "grpo clipped-ratio loss",
                 "group advantages"):
        assert part in proc.stdout
