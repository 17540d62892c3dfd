import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    """The product package (directory name has a hyphen, hence importlib)."""
    return importlib.import_module("pre-tjax_amd")


@pytest.fixture(scope="session")
def mt():
    return importlib.import_module("pre-tjax_amd.model_triton")


@pytest.fixture(scope="session")
def lo():
    return importlib.import_module("pre-tjax_amd.loss_and_optimizer_triton")
