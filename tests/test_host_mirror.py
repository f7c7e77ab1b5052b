"""Runs the C++ test of the host mirror (include/kvx.hpp, tests/cpp/kvx_host_test.cpp):
the reference's host-side known answers and error behaviour through the C++
classes that carry the reference's names."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "cpp", "kvx_host_test")


def _binary():
    if not os.path.exists(BINARY):
        from richengine_amd import build
        if not os.path.exists(build.LIB):
            build.build(verbose=False)
        build.build_host_test(verbose=False)
    return BINARY


def _run(mode):
    done = subprocess.run([_binary(), mode], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout + done.stderr
    assert f"kvx_host_test ({mode}): ok" in done.stdout


def test_host_mirror_known_answers():
    _run("host")


@pytest.mark.gpu
def test_host_mirror_on_device():
    _run("device")
