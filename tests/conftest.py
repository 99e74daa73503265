import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _have_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    # GPU tests are selected with -m gpu; if they get collected on a host without a GPU
    # (plain `pytest tests/`), skip them instead of failing in the HIP runtime.
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU on this host")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session", autouse=True)
def built_artifacts():
    """The tests load what is built; only where a build product is missing altogether (a fresh
    checkout) is it compiled here, once per session."""
    from ringattention_amd import _build
    if not os.path.exists(_build.LIB_PATH):
        _build.build_library()
    if not os.path.exists(_build.TORCH_LIB_PATH):
        _build.build_torch_shim()
    if not os.path.exists(_build.HARNESS_PATH):
        _build.build_harness()
    from oracle import build as oracle_build
    if not os.path.exists(oracle_build.LIB_PATH):
        oracle_build.build_oracle()


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.load()
    return o


@pytest.fixture(scope="session")
def ralib():
    from ringattention_amd import _lib
    return _lib.load()
