import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """The tests load the libraries that are built; only when there are none do they build."""
    pkg = os.path.join(ROOT, "graph_sampling_amd")
    if all(os.path.exists(os.path.join(pkg, name)) for name in ("libgs_hip.so", "libgs.so")):
        return
    from graph_sampling_amd import build
    build.build_all()


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")
