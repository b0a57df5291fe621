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


def test_probe_library_exports_every_symbol_of_its_header_and_the_backend_none_of_them():
    """Measurement and self-test code lives in libiomx_probe.so; libiomx.so holds operations and
    runtime only."""
    from iom_amd import iomx
    header = open(os.path.join(ROOT, "include", "iomx_probe.h")).read()
    declared = set(re.findall(r"\b(iomx_[a-z0-9_]+)\s*\(", header))
    assert declared == set(iomx.PROBE_SYMBOLS), declared ^ set(iomx.PROBE_SYMBOLS)
    probe = iomx.probe_lib()
    for name in sorted(declared):
        assert hasattr(probe, name), name
    exported = subprocess.check_output(["nm", "-D", "--defined-only", iomx.LIB_PATH]).decode()
    assert "probe" not in exported and "selftest" not in exported


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


def test_cxx_backend_links_nothing_of_the_checkers_or_of_the_cpu_backend():
    """The product library needs IOM's backend-independent layer (libiom.so, built beside it)
    and the kernel library, found next to itself; nothing under oracle/, and no symbol of the
    reference CPU backend."""
    path = os.path.join(ROOT, "iom_amd", "lib", "libiom_mi355x.so")
    if not os.path.exists(path):
        pytest.skip("C++ backend not built (needs the reference headers)")
    dynamic = subprocess.check_output(["readelf", "-d", path]).decode()
    needed = re.findall(r"\(NEEDED\)\s+Shared library: \[([^\]]+)\]", dynamic)
    assert "libiomx.so" in needed and "libiom.so" in needed
    assert not [n for n in needed if "oracle" in n or "core" in n or "cpu" in n or "ref" in n], needed
    runpath = re.findall(r"\((?:RUNPATH|RPATH)\)\s+Library (?:runpath|rpath): \[([^\]]*)\]", dynamic)
    assert runpath == ["$ORIGIN"], runpath
    undefined = subprocess.check_output(["nm", "-D", "--undefined-only", "-C", path]).decode()
    assert "iom::cpu" not in undefined and "make_cpu_device" not in undefined
    # the same holds for the layer it links: IOM's facade, without any backend
    facade = os.path.join(ROOT, "iom_amd", "lib", "libiom.so")
    defined = subprocess.check_output(["nm", "-D", "--defined-only", "-C", facade]).decode()
    assert "iom::DeviceOps::wait" in defined
    assert "make_cpu_device" not in defined and "iom::cpu" not in defined
    assert "oracle" not in subprocess.check_output(["readelf", "-d", facade]).decode()


def test_cxx_backend_exports_its_test_seams():
    path = os.path.join(ROOT, "iom_amd", "lib", "libiom_mi355x.so")
    if not os.path.exists(path):
        pytest.skip("C++ backend not built (needs the reference headers)")
    out = subprocess.check_output(["nm", "-D", "--defined-only", "-C", path]).decode()
    for name in ("iom::rocm_detail::inject_submission_fault_for_testing",
                 "iom::rocm_detail::queue_resource_snapshot_for_testing",
                 "iom::rocm_detail::reclaim_retained_queue_leases_for_testing",
                 "iom::rocm_detail::event_create_count_for_testing"):
        assert name in out, name
