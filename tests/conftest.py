import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm device (run with -m gpu on an MI355X box)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no ROCm device visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def golden():
    import numpy as np

    path = os.path.join(ROOT, "tests", "golden", "reference_vectors.npz")
    return dict(np.load(path, allow_pickle=False))


@pytest.fixture(scope="session")
def golden_next():
    """Vectors of the node types and layers added later (tests/golden/make_golden_next.py)."""
    import numpy as np

    path = os.path.join(ROOT, "tests", "golden", "reference_vectors_next.npz")
    return dict(np.load(path, allow_pickle=False))
