import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def rk():
    """The host package (directory ``amdgpu.jl_amd``), bound to the built librk.so."""
    from __graft_entry__ import load_package
    return load_package()


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    return oracle
