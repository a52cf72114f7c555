import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def strix():
    """The GPU library binding. Fails loudly when the HIP extension is missing or no GPU is present."""
    from __graft_entry__ import load_package
    pkg = load_package()
    pkg.require_gpu()
    return pkg
