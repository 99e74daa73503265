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
    """The tests load what is built.  A build product is compiled here, once per session, only where it
    is missing or was made from other sources than the ones in the tree (every build leaves a stamp
    with the hash of its sources): tests never run against a stale binary."""
    from ringattention_amd import _build
    if "RINGATTN_LIB" not in os.environ and not _build.is_current(_build.LIB_PATH, _build.library_sources()):
        _build.build_library()
    if not _build.is_current(_build.TORCH_LIB_PATH, _build.torch_shim_sources()):
        _build.build_torch_shim()
    if not _build.is_current(_build.HARNESS_PATH, _build.harness_sources()):
        _build.build_harness()
    from oracle import build as oracle_build
    if "ORACLE_LIB" not in os.environ and not oracle_build.is_current():
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
