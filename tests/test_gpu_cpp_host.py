"""The C++ host side (include/hpt_hip.hpp) on a device: runs the prebuilt test program
hpt_amd/lib/host_api_test (source tests/cpp/host_api_test.cpp, built by `python -m hpt_amd.build`)."""
import subprocess

import pytest

pytestmark = pytest.mark.gpu


def test_cpp_host_api_program():
    from hpt_amd import build
    assert build.HOST_TEST_BIN.exists(), f"{build.HOST_TEST_BIN} is missing: run `python -m hpt_amd.build`"
    r = subprocess.run([str(build.HOST_TEST_BIN)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, f"host_api_test failed:\n{r.stdout}\n{r.stderr}"
    assert " 0 failures" in r.stdout
