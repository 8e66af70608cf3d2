import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # the kernels are loaded from the in-tree build; compile only when nothing has been built yet
    from sla_amd import build as _build
    if not os.path.exists(_build.LIBPATH):
        _build.build(force=True)


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda:0")


def cos_sim(a, b):
    a = a.detach().double().flatten()
    b = b.detach().double().flatten()
    return float((a @ b) / (a.norm() * b.norm() + 1e-300))


def max_abs(a, b):
    return float((a.detach().double() - b.detach().double()).abs().max())


@pytest.fixture(autouse=True)
def _deterministic_seed():
    torch.manual_seed(1234)
