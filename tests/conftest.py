import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box with -m gpu)")


@pytest.fixture(scope="session")
def oracle_c():
    """The plain-C checker, built on demand (test infrastructure only)."""
    import ctypes
    import subprocess

    odir = os.path.join(ROOT, "oracle")
    so = os.path.join(odir, "libmuon_oracle.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", odir])
    lib = ctypes.CDLL(so)
    return lib


def pytest_terminal_summary(terminalreporter):
    """Parity figures the GPU tests measured (worst relative errors against the oracle), also in quiet runs."""
    from tests.helpers import PARITY_REPORT

    if PARITY_REPORT:
        terminalreporter.write_sep("-", "measured parity figures")
        for line in PARITY_REPORT:
            terminalreporter.write_line(line)
