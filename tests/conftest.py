import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run on the GPU box with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np
    return np.load(os.path.join(ROOT, "tests", "golden", "block_vectors.npz"), allow_pickle=False)


@pytest.fixture(scope="session")
def yahkv():
    """The product's Python binding (the package directory name has hyphens, so it is imported by name)."""
    import importlib
    return importlib.import_module("yet-another-halo-engine_amd")


@pytest.fixture(scope="session")
def torch_gpu():
    import torch
    assert torch.cuda.is_available(), "GPU tests need an MI355X"
    return torch
