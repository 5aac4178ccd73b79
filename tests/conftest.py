import os
import sys

import pytest

# the operator keeps the last view's sorted keys alive for the parity tests (read when the package is imported)
os.environ.setdefault("D3GS_KEEP_SORTED_KEYS", "1")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import d3gs_oracle
    d3gs_oracle.build()
    return d3gs_oracle
