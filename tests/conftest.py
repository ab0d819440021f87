import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    """The product package (directory `distributed-xfold_amd`, module
    `distributed_xfold_amd`)."""
    import __graft_entry__ as ge
    return ge.load_package()


@pytest.fixture(scope="session")
def gpu_pkg(pkg):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    pkg.lib.load()          # raises if the HIP library is missing: no fallback
    return pkg
