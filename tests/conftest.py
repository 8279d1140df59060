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


@pytest.fixture(autouse=True)
def _free_sparse_tables(request):
    """A sparse table keeps its HBM until the process ends (as the reference's tables keep their host
    memory); with the default size that is 17 GB per table, and one test needs 176 GB for its own.  So
    every GPU test gives back what the tables it created hold."""
    if request.node.get_closest_marker("gpu") is None:
        yield
        return
    import tensornet_amd.core as core

    created = []
    real = core.create_sparse_table

    def tracking(*args, **kwargs):
        h = real(*args, **kwargs)
        created.append(h)
        return h

    core.create_sparse_table = tracking
    try:
        yield
    finally:
        core.create_sparse_table = real
        for h in created:
            core.clear_sparse_table(h)
