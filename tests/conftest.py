"""Shared pytest setup: import paths, the `gpu` marker, and helpers used by the parity tests."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "ml-autofocusformer_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def device():
    return torch.device("cuda:0")


# tolerances of the parity bar: max|x-ref| / max|ref|
TOL = {torch.float32: 1e-5, torch.float64: 1e-12, torch.float16: 1e-2, torch.bfloat16: 1e-2}
TOL_SCATTER_F32 = 1e-4  # fp32 gradients that are accumulated by atomics in arbitrary order
