import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    import oracle as _oracle
    _oracle.lib()  # builds liboracle.so on first use if it is not there
    return _oracle


@pytest.fixture(scope="session")
def lib():
    import cuasr_amd
    if not os.path.exists(cuasr_amd.LIB_PATH):
        from cuasr_amd import build
        build.build()
    return cuasr_amd.load()
