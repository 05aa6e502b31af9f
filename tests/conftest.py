import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session", autouse=True)
def _built_libraries():
    """Load what is built; build only if nothing is."""
    from deserve_amd import _lib
    from oracle import c_oracle

    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    if not os.path.exists(os.path.join(ROOT, "oracle", "libkv_oracle.so")):
        c_oracle.build()
