import os
import sys

import pytest

REPO_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO_ROOT not in sys.path:
    sys.path.insert(0, REPO_ROOT)
TESTS_DIR = os.path.dirname(os.path.abspath(__file__))
if TESTS_DIR not in sys.path:
    sys.path.insert(0, TESTS_DIR)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    # a fresh checkout holds no built libraries (they are not under version control): build them once
    import __graft_entry__

    __graft_entry__.ensure_built()


@pytest.fixture(scope="session")
def gpu():
    """Session-wide handle for GPU tests: fails loudly (no skip, no fallback) when the HIP
    library or the device is missing."""
    import torch
    from nnforge_amd import capi

    lib = capi.load()
    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    import nnf_testing

    return nnf_testing.GpuHarness(lib)
