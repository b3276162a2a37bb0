"""Builds libclahip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libclahip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-ffp-contract=off", "-munsafe-fp-atomics",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def build_lib(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", LIB] + sources()
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


HOST_DIR = os.path.join(HERE, "host")
HOST_LIB = os.path.join(HOST_DIR, "_clahost.so")


def build_host(verbose=True):
    """The C++ host layer (host/cla_host.hpp) as a Python module over libclahip.so."""
    import sysconfig
    import pybind11
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall",
           "-I" + sysconfig.get_paths()["include"], "-I" + pybind11.get_include(),
           os.path.join(HOST_DIR, "bindings.cpp"), "-o", HOST_LIB,
           "-L" + HERE, "-lclahip", "-Wl,-rpath,$ORIGIN/.."]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return HOST_LIB


if __name__ == "__main__":
    build_lib()
    build_host()
    sys.exit(0)
