"""The C ABI driven from plain C (tests/cla_c_driver.c, built by systemds_amd/build.py): block construction from
C arrays, the four products, decompression and counts, each checked inside the driver against long-double
products of the dense matrix it built. This is the call pattern of a JNI shim (systemds_amd/jni/cla_jni.c),
with no Python or C++ between the caller and include/cla_hip.h."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

DRIVER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cla_c_driver")


@pytest.mark.parametrize("n_rows", [1, 4097, 300007])
def test_c_driver(n_rows):
    assert os.path.exists(DRIVER), "tests/cla_c_driver not built: run __graft_entry__.build()"
    r = subprocess.run([DRIVER, str(n_rows)], capture_output=True, text=True, timeout=170)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "C-DRIVER OK" in r.stdout and "FAIL" not in r.stdout
