"""Builds the native libraries of the package in-tree.

  lib/libttmlir_amd_hip.so   gfx950 kernels + C ABI (csrc/*.hip, hipcc)
  lib/libttmlir_amd_rt.so    C++ host runtime in the tt::runtime style (runtime/*.cpp, g++)

Usage: python build.py [--force] [--jobs N]
"""
import argparse
import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
RTSRC = os.path.join(HERE, "runtime")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
INCLUDE = os.path.join(ROOT, "include")

HIP_LIB = os.path.join(LIBDIR, "libttmlir_amd_hip.so")
RT_LIB = os.path.join(LIBDIR, "libttmlir_amd_rt.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unknown-attributes", "-Wno-unused-command-line-argument",
    "-I", INCLUDE, "-I", CSRC,
]
CXX = os.environ.get("CXX", "g++")
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wextra", "-pthread",
             "-I", INCLUDE, "-I", RTSRC]


def _newer(target, deps):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def _compile(job):
    src, obj, cmd, deps, force = job
    if not force and _newer(obj, [src] + deps):
        return obj, ""
    return obj, _run(cmd + ["-c", src, "-o", obj])


def build_hip(force=False, jobs=8, verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    hdrs = sorted(glob.glob(os.path.join(CSRC, "*.h"))) + sorted(glob.glob(os.path.join(INCLUDE, "*.h")))
    work = [(s, os.path.join(OBJDIR, os.path.basename(s) + ".o"), [HIPCC] + HIP_FLAGS, hdrs, force) for s in srcs]
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for obj, out in ex.map(_compile, work):
            objs.append(obj)
            if verbose and out.strip():
                print(out)
    if force or not _newer(HIP_LIB, objs):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIB] + objs)
    return HIP_LIB


def build_runtime(force=False, jobs=8, verbose=True):
    srcs = sorted(glob.glob(os.path.join(RTSRC, "*.cpp")))
    if not srcs:
        return None
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    hdrs = sorted(glob.glob(os.path.join(RTSRC, "*.h"))) + sorted(glob.glob(os.path.join(INCLUDE, "*.h")))
    work = [(s, os.path.join(OBJDIR, os.path.basename(s) + ".o"), [CXX] + CXX_FLAGS, hdrs, force) for s in srcs]
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for obj, out in ex.map(_compile, work):
            objs.append(obj)
            if verbose and out.strip():
                print(out)
    if force or not _newer(RT_LIB, objs):
        _run([CXX, "-shared", "-fPIC", "-pthread", "-o", RT_LIB] + objs +
             ["-L", LIBDIR, "-lttmlir_amd_hip", "-Wl,-rpath,$ORIGIN", "-ldl"])
    return RT_LIB


def build_all(force=False, jobs=8, verbose=True):
    return build_hip(force, jobs, verbose), build_runtime(force, jobs, verbose)


def clean():
    shutil.rmtree(OBJDIR, ignore_errors=True)
    for p in (HIP_LIB, RT_LIB):
        if os.path.exists(p):
            os.remove(p)


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--jobs", type=int, default=8)
    ap.add_argument("--clean", action="store_true")
    a = ap.parse_args()
    if a.clean:
        clean()
        sys.exit(0)
    print(build_all(a.force, a.jobs))
