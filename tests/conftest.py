import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box only)")


@pytest.fixture(scope="session")
def port():
    """The C restatement of the CpuRef hot path (built on demand: plain gcc, seconds)."""
    from oracle import cpuref
    if not cpuref.have("port"):
        cpuref.build(reference=False)
    return cpuref.Oracle("port")


@pytest.fixture(scope="session")
def reference():
    """The reference's own hot-path sources compiled by oracle/Makefile (skipped where it is not built)."""
    from oracle import cpuref
    if not cpuref.have("reference"):
        if os.path.isdir("/root/reference/src/backends/reference"):
            cpuref.build(reference=True)
        else:
            pytest.skip("oracle/_ref is not built and the reference tree is not mounted")
    return cpuref.Oracle("reference")
