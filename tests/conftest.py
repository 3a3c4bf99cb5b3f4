import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "fused-swiglu_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # GPU tests are selected explicitly with -m gpu; without a GPU they are skipped rather than failed.
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def capi():
    import fsw_capi
    fsw_capi.lib()  # raises if libfsw_hip.so is missing: no fallback
    return fsw_capi


@pytest.fixture(scope="session")
def ext():
    import fused_mlp_module  # raises if the extension is not built: no fallback
    return fused_mlp_module
