"""Builds libclahip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Every .hip file under csrc/ is compiled to an object of its own (in parallel) and the
objects are linked into one shared library. `python -m systemds_amd.build --incremental`
recompiles only the files that are newer than their object (development); the default
and `__graft_entry__.build()` compile everything.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "obj")
LIB = os.path.join(HERE, "libclahip.so")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-ffp-contract=off", "-munsafe-fp-atomics",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    hs += [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE) if f.endswith(".h")]
    return hs


def build_lib(verbose=True, incremental=False, jobs=None):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ, exist_ok=True)
    newest_header = max(os.path.getmtime(h) for h in _headers())
    jobs = jobs or min(8, os.cpu_count() or 1)

    def compile_one(src):
        obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
        if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header):
            return obj
        cmd = [hipcc] + HIPCC_FLAGS + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, sources()))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
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


ROOT = os.path.dirname(HERE)
C_DRIVER = os.path.join(ROOT, "tests", "cla_c_driver")


def build_c_driver(verbose=True):
    """The plain-C test driver of the C ABI (tests/cla_c_driver.c), linked against libclahip.so."""
    cc = os.environ.get("CC", "gcc")
    cmd = [cc, "-O2", "-std=gnu11", "-Wall", "-Wextra", "-I" + INCLUDE, C_DRIVER + ".c", "-o", C_DRIVER,
           "-L" + HERE, "-lclahip", "-Wl,-rpath,$ORIGIN/../systemds_amd", "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return C_DRIVER


def build_jni(verbose=True):
    """The JNI shim (jni/cla_jni.c) when a JDK is present ($JAVA_HOME/include/jni.h); returns None otherwise."""
    jh = os.environ.get("JAVA_HOME")
    if not jh or not os.path.exists(os.path.join(jh, "include", "jni.h")):
        return None
    out = os.path.join(HERE, "libclahip_jni.so")
    cmd = [os.environ.get("CC", "gcc"), "-O2", "-fPIC", "-shared", "-I" + os.path.join(jh, "include"),
           "-I" + os.path.join(jh, "include", "linux"), "-I" + INCLUDE, os.path.join(HERE, "jni", "cla_jni.c"), "-o", out,
           "-L" + HERE, "-lclahip", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    build_lib(incremental="--incremental" in sys.argv)
    if "--no-host" not in sys.argv:
        build_host()
        build_c_driver()
        build_jni()
    sys.exit(0)
