import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


BUILD_MODE = "unknown"


def pytest_sessionstart(session):
    """The tests load the libraries that are built, as long as they were built from the sources
    as they are now (the build leaves a hash of csrc/ and include/ beside them); when the
    libraries are missing or stale they are built first."""
    global BUILD_MODE
    from graph_sampling_amd import build
    state = build.build_state()
    if state == "current":
        BUILD_MODE = "prebuilt libraries, source hash %s" % build.source_hash()[:16]
    elif state == "unknown":
        BUILD_MODE = "prebuilt libraries with no source hash beside them (not rebuilt)"
    else:
        build.build_all()
        BUILD_MODE = "%s libraries: built at session start, source hash %s" % (
            state, build.source_hash()[:16])


def pytest_report_header(config):
    return "graph_sampling_amd native libraries: " + BUILD_MODE


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")
