"""CPU-side checks of the shipped libraries: they load and export every declared
symbol.  No compute call is made (there is no GPU here)."""
import ctypes as C
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_libiomx_exports_every_symbol_of_the_header():
    from iom_amd import iomx
    header = open(os.path.join(ROOT, "include", "iomx.h")).read()
    declared = set(re.findall(r"\b(iomx_[a-z0-9_]+)\s*\(", header))
    assert declared == set(iomx.SYMBOLS), declared ^ set(iomx.SYMBOLS)
    lib = iomx.lib()
    for name in sorted(declared):
        assert hasattr(lib, name), name
    assert lib.iomx_error_string(-1).decode().startswith("iomx")


def test_status_queries_do_not_need_a_gpu():
    from iom_amd import iomx
    assert iomx.device_count() >= 0
    info = iomx.LaunchInfo()
    assert iomx.lib().iomx_last_launch(C.byref(info)) == 0


def test_cxx_backend_exports_the_factory():
    path = os.path.join(ROOT, "iom_amd", "lib", "libiom_mi355x.so")
    if not os.path.exists(path):
        pytest.skip("C++ backend not built (needs the reference headers)")
    out = subprocess.check_output(["nm", "-D", "--defined-only", "-C", path]).decode()
    assert "iom::make_rocm_device(unsigned int, iom::DeviceMemoryConfig, iom::QueueConfig)" in out
    # the backend reaches HIP only through the C ABI
    undefined = subprocess.check_output(["nm", "-D", "--undefined-only", path]).decode()
    assert "iomx_launch_binary" in undefined
    assert not re.search(r"\bhip[A-Z]", undefined)
