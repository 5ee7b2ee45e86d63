import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")

# the tests load what is built; only a tree in which nothing is built gets compiled here
import __graft_entry__  # noqa: E402
__graft_entry__.ensure_built()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def zfp_golden():
    return np.load(os.path.join(GOLDEN, "zfp_golden.npz"))


@pytest.fixture(scope="session")
def torch_golden():
    return np.load(os.path.join(GOLDEN, "torch_golden.npz"))


def case(golden, name):
    return {k[len(name) + 1:]: golden[k] for k in golden.files if k.startswith(name + ".")}
