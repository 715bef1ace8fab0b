"""The C++ host side above the C ABI (include/mummu_moe.hpp), driven by its own test program
(tests/cpp/host_mirror_test.cpp), which restates the reference's unit tests of the block
(nn/moe.rs:1655-1700, 1976-1979, 2177-2202, 2340-2352; experts.rs:1365-1417)."""
import os
import subprocess

import pytest

from mummu_amd import build

BIN = build.HOST_TEST_BIN


def _binary():
    if not os.path.exists(BIN):
        build.build_host_mirror_test()
    return BIN


def test_host_mirror_config_validation_needs_no_gpu():
    r = subprocess.run([_binary(), "--no-gpu"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok" in r.stdout


@pytest.mark.gpu
def test_host_mirror_reference_unit_tests():
    r = subprocess.run([_binary()], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "host mirror: ok" in r.stdout
