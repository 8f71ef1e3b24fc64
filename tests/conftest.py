import hashlib
import pathlib
import random
import sys

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with `-m gpu` on the GPU box)")


def _seed_for(text):
    return int(hashlib.sha256(text.encode("utf-8")).hexdigest(), 16) % 2**32


@pytest.fixture(autouse=True)
def seed_per_test(request):
    """Every test gets inputs that depend only on its id (the reference seeds
    the same way, tests/conftest.py:8-37 of the reference)."""
    import numpy as np
    import torch

    seed = _seed_for(request.node.nodeid)
    random.seed(seed)
    np.random.seed(seed % 2**32)
    torch.manual_seed(seed)
    yield
