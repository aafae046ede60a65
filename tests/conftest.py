import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture
def make_model():
    """Models created through this fixture are unloaded after the test
    (the reference's tests/features/conftest.py:7-19 does the same)."""
    created = []

    def _make(*args, **kwargs):
        from genn_amd.genn_model import GeNNModel
        m = GeNNModel(*args, **kwargs)
        created.append(m)
        return m

    yield _make
    for m in created:
        m.unload()
