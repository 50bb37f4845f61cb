import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session", autouse=True)
def _oracle_threads():
    """The oracle is bit-identical for any thread count; use the cores we have for speed."""
    from oracle import cpu_ref
    cpu_ref.set_threads(min(8, os.cpu_count() or 1))
    yield
