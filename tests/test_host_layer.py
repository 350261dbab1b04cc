"""Runs the C++ host operator layer's own test program (qwegn_amd/host/host_tests.cpp): the mirror of the
reference's QWGemm / QWGemmAQ / QWMoEOperator API above the C ABI."""
import os
import subprocess

import pytest

from qwegn_amd import build as qbuild


def _exe():
    if not qbuild.HOST_TESTS.exists():
        qbuild.build_host_tests()
    return str(qbuild.HOST_TESTS)


def test_host_layer_cpu_checks():
    mode = "--cpu" if os.path.exists("/dev/kfd") else "--cpu-nodevice"
    res = subprocess.run([_exe(), mode], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "0 failed" in res.stdout


@pytest.mark.gpu
def test_host_layer_on_device():
    res = subprocess.run([_exe(), "--gpu"], capture_output=True, text=True, timeout=300)
    print(res.stdout)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "0 failed" in res.stdout
