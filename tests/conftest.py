import importlib
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    """The product package (its directory name is not a Python identifier)."""
    return importlib.import_module("text-generation-inference_amd")


@pytest.fixture(scope="session")
def oracle():
    from oracle import q4_oracle

    return q4_oracle


@pytest.fixture(scope="session")
def gpu(pkg):
    """Session fixture of the GPU tests: torch on cuda:0 with the built library loaded."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    pkg._lib.load()  # fail loudly here if the library was not built
    torch.cuda.set_device(0)
    return torch.device("cuda:0")
