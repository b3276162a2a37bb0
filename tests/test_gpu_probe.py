"""The device probe (systemds_amd/probe/cla_probe.hip, built by systemds_amd/build.py): the operand layout of
v_mfma_f64_4x4x4_f64 that k_rmm_mfma and the narrow block of k_tsmm_decode assume holds on this device, and the
probe's rate loops run to the end."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

PROBE = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "systemds_amd", "cla_probe")


def test_probe_runs_and_the_matrix_instruction_layout_is_the_assumed_one():
    assert os.path.exists(PROBE), "systemds_amd/cla_probe not built: run __graft_entry__.build()"
    r = subprocess.run([PROBE], capture_output=True, text=True, timeout=110)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "layout of v_mfma_f64_4x4x4_f64: as assumed" in r.stdout
    rates = [float(x) for x in re.findall(r"([0-9.]+) TB/s", r.stdout)]
    assert len(rates) >= 10 and all(x > 0.1 for x in rates)
    assert "sums in vector registers, two waves per SIMD" in r.stdout and "on the SIMD's other wave" in r.stdout
