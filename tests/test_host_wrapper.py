"""The C++ host wrapper over the C ABI (nerva_amd/host/nerva_hip.hpp), compiled with g++ against
libnerva_hip.so and run as a small program: validation and no-device behaviour on the CPU, the
reference's greedy-stream known-answer model on the GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBDIR = os.path.join(ROOT, "nerva_amd")
BIN = os.path.join(ROOT, "tests", "host", "host_wrapper_check")


def build():
    """Compiles the check program when a C++ compiler is here; otherwise uses the one already built."""
    cxx = shutil.which("g++")
    if cxx is None:
        assert os.path.exists(BIN), "no g++ and no prebuilt host_wrapper_check"
        return BIN
    rocm_lib = "/opt/rocm/lib"
    cmd = [cxx, "-std=c++17", "-O1", "-Wall", "-Wextra", "-I" + os.path.join(ROOT, "include"),
           "-I" + os.path.join(LIBDIR, "host"), os.path.join(ROOT, "tests", "host", "host_wrapper_check.cpp"),
           "-L" + LIBDIR, "-lnerva_hip", "-Wl,-rpath," + LIBDIR, "-Wl,-rpath," + rocm_lib,
           "-Wl,-rpath-link," + rocm_lib, "-o", BIN]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stdout + res.stderr
    return BIN


def run(mode):
    res = subprocess.run([build(), mode], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "0 failure(s)" in res.stdout


def test_host_wrapper_validation_and_no_device_behaviour():
    run("cpu")


@pytest.mark.gpu
def test_host_wrapper_reference_greedy_stream():
    run("gpu")
