import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PKG = "marian-dev_amd"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def load(name=None):
    """Import the package (its directory name has a hyphen) or one of its modules."""
    return importlib.import_module(PKG if name is None else PKG + "." + name)


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def synth():
    return load("synth")


@pytest.fixture(scope="session")
def integer():
    """Host mirror on the GPU; fails loudly when the HIP library or the GPU is missing."""
    import torch
    assert torch.cuda.is_available(), "gpu tests need a GPU"
    mod = load("integer")
    load("_lib").lib()
    return mod
