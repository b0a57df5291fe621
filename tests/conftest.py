"""Test configuration: the `gpu` marker and import paths.

CPU tests (`-m "not gpu"`) pin the oracle and check that the C-ABI library
loads and exports every declared symbol.  GPU tests (`-m gpu`) are the parity
tests proper: they call the HIP path through the C-ABI and compare with the
oracle, the compiled reference where it was built, and the golden fixtures.
"""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def ref():
    """The compiled reference CPU backend, where oracle/_ref was built."""
    import iomo
    if not iomo.ref_available():
        pytest.skip("oracle/_ref/libiom_ref.so not built (needs the reference sources)")
    backend = iomo.ref_backend()
    yield backend
    backend.close()
