import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def O():
    """The CPU oracle."""
    return entry.load_oracle()


@pytest.fixture(scope="session")
def pkg():
    return entry.load_package()


@pytest.fixture(scope="session")
def B(pkg):
    return pkg.binding


@pytest.fixture(scope="session")
def L(pkg):
    return pkg.layout


@pytest.fixture(scope="session")
def host(pkg):
    return importlib.import_module(entry.PKG_NAME + ".host")


@pytest.fixture(scope="session")
def torch_gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test on a machine without a GPU")
    return torch
