"""Runs the C++ API test programs (tests/cxx): the reference's own DIA test
cases re-expressed against the C++ mirror headers.  test_dia_host needs no GPU;
test_dia_gpu drives the HIP kernels through the headers and the C ABI."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CXX = os.path.join(HERE, "cxx")


def _binary(name):
    path = os.path.join(CXX, "bin", name)
    if not os.path.exists(path):
        # not built yet: build in-tree (the driver's build() normally did this)
        root = os.path.dirname(HERE)
        if not os.path.exists(os.path.join(root, "cuv_amd", "lib", "libcuvdia.so")):
            subprocess.check_call(["make", "-C", os.path.join(root, "cuv_amd", "csrc")])
        subprocess.check_call(["make", "-C", os.path.join(root, "oracle")])
        subprocess.check_call(["make", "-C", CXX])
    return path


def _run(name):
    p = subprocess.run([_binary(name)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    print(p.stdout)
    assert p.returncode == 0, p.stdout[-4000:]
    assert "0 failure(s)" in p.stdout


def test_cxx_host_side():
    _run("test_dia_host")


@pytest.mark.gpu
def test_cxx_device_side():
    _run("test_dia_gpu")
