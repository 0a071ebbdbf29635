"""The C ABI driven from plain C++ (vortex_amd/csrc/abi_selftest.cpp): no torch, no Python in the process."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu


def test_cpp_selftest_passes():
    from vortex_amd import _lib, build
    if not os.path.exists(build.SELFTEST):
        pytest.fail("vortex_amd/abi_selftest is not built; run python -m vortex_amd.build")
    r = subprocess.run([build.SELFTEST, _lib.LIB_PATH], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=120)
    assert r.returncode == 0 and "abi_selftest: ok" in r.stdout, r.stdout
