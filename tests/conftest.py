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


# Worst errors that the GPU tests saw, by label: printed after the run, so that the bounds of the
# bfloat16 comparisons can be held near what is observed (about twice the worst) and not at a
# flat guess.
OBSERVED = {}


def observe(label, value):
    OBSERVED[label] = max(OBSERVED.get(label, 0.0), float(value))


def pytest_terminal_summary(terminalreporter):
    if OBSERVED:
        terminalreporter.write_line("observed errors (worst per label):")
        for label in sorted(OBSERVED):
            terminalreporter.write_line(f"  {label}: {OBSERVED[label]:.5g}")
