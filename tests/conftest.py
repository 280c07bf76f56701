import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on a GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def cpu_ops(monkeypatch):
    """Replaces the HIP kernels by their plain torch references, so that the engine's host logic
    (step function, cache bookkeeping, scheduler) can be exercised without a GPU.  Tests only."""
    import torch_ops
    from simply_amd.kernels import ops

    for name in ("embed", "rmsnorm", "add_rmsnorm", "rope_cache_write", "rope", "gather_rows", "fill_", "gemm",
                 "paged_attention", "sample", "score", "decode_attention_takes"):
        monkeypatch.setattr(ops, name, getattr(torch_ops, name))
    return torch_ops


@pytest.fixture(scope="session")
def gpu_lib():
    """The built kernel library; GPU tests fail loudly if it is not there."""
    from simply_amd.kernels import lib

    lib.load()
    assert lib.library_path() is not None
    return lib
