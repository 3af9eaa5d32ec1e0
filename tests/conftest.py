import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def be():
    """One backend for the whole GPU session (the reference's sweep_linear_on does the same for
    backends without an address-keyed weight cache, crates/infr-testkit/src/lib.rs:462-476)."""
    from infr_amd import HipBackend
    b = HipBackend(0)
    yield b
    b.close()
