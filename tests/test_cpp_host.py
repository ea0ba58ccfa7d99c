"""C++ translation units compiled and run on the host (no GPU): the device pool's bookkeeping with a mock driver, and the
integration sketches of INTEGRATION.md compiled against the public headers."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")
RT = os.path.join(ROOT, "tt-mlir_amd", "runtime")
INC = os.path.join(ROOT, "include")


def compile_cpp(tmp_path, name, extra=()):
    exe = str(tmp_path / name)
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-pthread", "-I", RT, "-I", INC,
           os.path.join(CPP, name + ".cpp"), "-o", exe] + list(extra)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    return exe


def test_device_pool_bookkeeping(tmp_path):
    exe = compile_cpp(tmp_path, "test_device_pool")
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert r.returncode == 0, r.stdout
