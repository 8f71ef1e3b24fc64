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


@pytest.fixture(autouse=True, scope="session")
def caches_in_a_temporary_directory(tmp_path_factory):
    """Tuned choices and kernel descriptions go to a directory of this test session, not to the
    home directory: what one run found does not steer the next, and nothing is left behind."""
    import importlib

    from ninetoothed_amd import auto_tuner

    make = importlib.import_module("ninetoothed_amd.make")  # (the package attribute `make` is the function)

    root = tmp_path_factory.mktemp("ninetoothed_amd_cache")
    saved = auto_tuner.CACHE_DIR, make.CACHE_DIR
    auto_tuner.CACHE_DIR, make.CACHE_DIR = root / "auto_tuning", root
    yield root
    auto_tuner.CACHE_DIR, make.CACHE_DIR = saved
