"""Runs the C++ host-layer tests (tests/cpp/host_api_test.cc): the reference-style operator API
over the C ABI.  The driver is built in-tree beforehand (build() or tests/cpp/build.py)."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "bin", "host_api_test")


def _binary():
    if not os.path.isfile(BIN):
        import importlib.util
        spec = importlib.util.spec_from_file_location("cpp_build", os.path.join(HERE, "cpp", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build()
    return BIN


def test_host_logic_on_cpu():
    out = subprocess.run([_binary(), "cpu"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert out.returncode == 0, out.stdout


@pytest.mark.gpu
def test_operators_through_device_hip():
    out = subprocess.run([_binary(), "gpu"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert out.returncode == 0, out.stdout
