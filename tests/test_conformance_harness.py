"""The assertion harness the conformance binary is compiled with (tests/conformance/doctest/doctest.h)
must itself report failures: tests/conformance/doctest_selftest.cpp holds cases built to fail and
checks the harness's counts and messages.  CPU only; compiled here if the build step has not."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CONF = os.path.join(ROOT, "tests", "conformance")
BINARY = os.path.join(ROOT, "oracle", "_ref", "doctest_selftest")


def test_harness_counts_failures_and_leaves_on_require(tmp_path):
    binary = BINARY
    if not os.path.exists(binary):
        if shutil.which("g++") is None:
            pytest.skip("no g++ to compile the harness self-test")
        binary = str(tmp_path / "doctest_selftest")
        subprocess.check_call(["g++", "-std=c++20", "-O1", "-I", CONF, "-o", binary,
                               os.path.join(CONF, "doctest_selftest.cpp")])
    proc = subprocess.run([binary], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert proc.returncode == 0 and "WRONG" not in proc.stdout, proc.stdout
    assert proc.stdout.count("\nok:") + proc.stdout.startswith("ok:") == 15
