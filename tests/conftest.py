import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import cpu

    cpu.load()
    return cpu


@pytest.fixture(scope="session")
def tn():
    """The product package with its HIP library loaded and a GPU present."""
    import torch

    import tensornet_amd

    tensornet_amd.load()
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import tensornet_amd.ops  # noqa: F401

    return tensornet_amd
