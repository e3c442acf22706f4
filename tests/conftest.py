import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.lib()
    return O


def pytest_collection_modifyitems(config, items):
    """PyTorch ships a HIP runtime of its own.  In a process that uses both, torch must be loaded before
    libturbovec_hip.so (which then binds to torch's copy); the other way round the process holds two runtimes
    and torch finds no GPU.  So a run that selects GPU tests imports torch before any of them loads the library."""
    if any(item.get_closest_marker("gpu") for item in items):
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
