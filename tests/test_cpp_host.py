"""C++ translation units compiled and run on the host (no GPU): the device pool's bookkeeping with a mock driver, and the
sketches of how the reference's runtime would bind this one, compiled against the public headers."""
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


def test_runtime_arm_sketch_compiles_and_runs(tmp_path):
    """The fourth arm of the reference's runtime dispatch: include/ttmlir_amd_runtime_arm.hpp over the C ABI, in its own namespace,
    linked against the exported ttrt_* symbols only."""
    import sys
    sys.path.insert(0, ROOT)
    import __graft_entry__ as entry
    entry.load_package()
    from ttmlir_amd import programs, runtime as rt
    rt.lib()
    path = tmp_path / "c1.ttnn"
    path.write_bytes(programs.c1_matmul())
    libdir = os.path.join(ROOT, "tt-mlir_amd", "lib")
    exe = compile_cpp(tmp_path, "test_runtime_arm", ["-L", libdir, "-lttmlir_amd_rt", "-Wl,-rpath," + libdir])
    r = subprocess.run([exe, str(path)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert r.returncode == 0, r.stdout
    assert "programs=1 inputs=2 layout=(0,0,2)" in r.stdout, r.stdout      # host, row-major, bf16 inputs of config 1
