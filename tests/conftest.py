import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PKG = "comfyui-backend-but-rust_amd"


def pkg(sub=None):
    """The package directory name has hyphens, so it is imported by string."""
    return importlib.import_module(PKG if sub is None else PKG + "." + sub)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """Without a GPU the `gpu` tests are skipped rather than failing in their first device call."""
    try:
        import torch
        have = torch.cuda.is_available()
    except ImportError:
        have = False
    if have:
        return
    skip = pytest.mark.skip(reason="needs a GPU")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def synth():
    return pkg("synth")
