import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    """The host-side package (its directory name has a hyphen, so no plain `import`)."""
    return importlib.import_module("llama-rust_amd")


@pytest.fixture(scope="session")
def lib(pkg):
    """The C-ABI shared library; fails loudly when it has not been built."""
    return pkg.load_library()
