import os
import sys

import pytest
import torch

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def host_pool_factory():
    """Host-memory stand-in for the fine-grained heap, for tests of the host
    logic on a machine without a GPU."""
    return lambda nbytes: torch.zeros(nbytes, dtype=torch.int8)


@pytest.fixture(scope="session")
def shmem_gpu():
    """One 6 GiB, 8-virtual-rank context shared by the GPU tests (the heap is
    a bump allocator that never frees, so tests reset its offset)."""
    import iris_amd

    ctx = iris_amd.iris(768 << 20, virtual_ranks=8)
    return ctx


@pytest.fixture()
def shmem(shmem_gpu):
    shmem_gpu.heap_offset = 0
    yield shmem_gpu
    torch.cuda.synchronize()
