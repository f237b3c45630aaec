import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.nx_oracle import OracleBackend

    return OracleBackend()


@pytest.fixture(scope="session")
def hip():
    """The HIP backend on cuda:0; fails (not skips) when the library is absent."""
    from raven_amd.nx_backend import Backend

    return Backend()
