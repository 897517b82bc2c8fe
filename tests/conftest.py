import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_built():
    """Build oracle/libscn_oracle.so on first use (plain g++, a few seconds)."""
    import subprocess
    so = os.path.join(ROOT, "oracle", "libscn_oracle.so")
    src = os.path.join(ROOT, "oracle", "scn_oracle.cpp")
    if not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "libscn_oracle.so"])
    return so
