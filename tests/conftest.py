import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ctx():
    """The one HipContext of the test session.  Fails loudly when the HIP library or the GPU
    is missing: GPU tests must never pass on a fallback."""
    from webdnn_amd import hostops

    context = hostops.HipContext(0).initialize()
    from oracle import ref

    ref.set_threads(min(16, os.cpu_count() or 1))
    return context


@pytest.fixture(autouse=True)
def _oracle_threads():
    from oracle import ref

    ref.set_threads(min(16, os.cpu_count() or 1))
    yield
