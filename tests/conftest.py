import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def olib():
    import oracle
    return oracle.lib()


@pytest.fixture(scope="session")
def hiplib():
    """The HIP kernel library through its C ABI; GPU tests fail (not skip) when it is not built."""
    import harness
    return harness.pkg.load_library()


@pytest.fixture(scope="session")
def probelib():
    """The measurement / verification aids (roofline probes, quantiser enumeration): a library of their own."""
    import harness
    return harness.pkg.load_probe_library()
