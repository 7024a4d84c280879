"""Runs the C++ test driver of the host-side TFCC layer (tests/cpp/host_tests.cpp).  The CPU part
exercises Shape / Variable / View / FlexAllocator and the argument checks on a host-memory device;
the GPU part runs the reference's data / blas / quantization cases on the ROCm device."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "wechat-tfcc_amd", "host", "build", "host_tests")


def _run(mode):
    if not os.path.exists(DRIVER):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "wechat-tfcc_amd", "csrc")])
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "wechat-tfcc_amd", "host")])
    res = subprocess.run([DRIVER, mode], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(res.stdout)
    assert res.returncode == 0, res.stdout[-4000:]
    assert "0 failures" in res.stdout


def test_host_layer_framework_cpu():
    _run("cpu")


@pytest.mark.gpu
def test_host_layer_gpu():
    _run("gpu")
