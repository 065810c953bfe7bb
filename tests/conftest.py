import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "experiments-pytorch-cuda-extension-for-sparse-matmul_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


def pytest_sessionstart(session):
    """The tests load the libraries that are built; only when nothing is built do they build (hipcc
    cross-compiles for gfx950 without a GPU).  The package itself never builds: it fails to import."""
    if not os.path.exists(os.path.join(PKG, "csrc", "libbsa_hip.so")):
        sys.path.insert(0, os.path.join(PKG, "csrc"))
        import build as csrc_build
        csrc_build.build(force=True)


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
