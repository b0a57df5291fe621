"""Builds tests/host_checks/leaves_host_check.cpp with hipcc (host side only runs) and
runs it: the tile-row packing helpers and the per-element arithmetic of the every-leaf
kernels, executed on the CPU against the oracle, with no device involved."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not available")
def test_leaf_arithmetic_and_packing_on_the_host(tmp_path):
    oracle = os.path.join(ROOT, "oracle")
    if not os.path.exists(os.path.join(oracle, "libiom_oracle.so")):
        pytest.skip("oracle/libiom_oracle.so not built")
    exe = str(tmp_path / "leaves_host_check")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-ffp-contract=off", "-w",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "iom_amd", "csrc"),
           "-I" + oracle, os.path.join(ROOT, "tests", "host_checks", "leaves_host_check.cpp"),
           "-o", exe, "-L" + oracle, "-liom_oracle", "-Wl,-rpath," + oracle]
    build = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert build.returncode == 0, build.stderr[-2000:]
    run = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stdout[-2000:]
    assert "TOTAL mismatches: 0" in run.stdout
