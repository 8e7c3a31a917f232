import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run on the GPU box)")


@pytest.fixture(scope="session")
def model_root(tmp_path_factory):
    """Temporary folder that holds the model folders the tests make."""
    return tmp_path_factory.mktemp("models")
