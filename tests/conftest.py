import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PKG_NAME = "tensor-program-optimization-with-auto-batching_amd"


def load_pkg(sub: str = ""):
    """Import the (hyphenated) package or one of its submodules."""
    return importlib.import_module(PKG_NAME + (("." + sub) if sub else ""))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def mlora():
    return load_pkg()


@pytest.fixture(scope="session")
def ops():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return load_pkg("ops")


@pytest.fixture(scope="session")
def synth():
    return load_pkg("synth")
