import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture
def rng():
    return np.random.default_rng(1234)


@pytest.fixture(scope="session")
def oracle_backend():
    from oracle.oracle_backend import OracleBackend
    return OracleBackend()


@pytest.fixture(scope="session")
def hip_backend():
    from honeycrisp_amd.backend import HIPBackend
    backend = HIPBackend()
    yield backend
    backend.sync()
    if os.environ.get("HCHIP_BATCHING"):   # a run of the whole suite with batching on: say how much of it was batched
        print("\nHCHIP_BATCHING=%s: launches listed / enqueued: %d / %d"
              % ((os.environ["HCHIP_BATCHING"],) + backend.batchingStats()))


class _Switches:
    """The library's measurement / test switches on the session's context (hc_debug_set), with
    monkeypatch's method names; whatever a test sets is back at its default when the test ends."""

    def __init__(self, backend):
        self.backend, self.touched = backend, set()

    def setenv(self, name, value):
        self.backend.debugSet(name, value)
        self.touched.add(name)

    def delenv(self, name):
        self.backend.debugSet(name, None)

    def restore(self):
        for name in self.touched:
            self.backend.debugSet(name, None)


@pytest.fixture
def switch(hip_backend):
    s = _Switches(hip_backend)
    yield s
    s.restore()
