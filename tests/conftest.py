import os
import sys

import pytest
import torch  # noqa: F401  (the tests compare against PyTorch on the CPU and borrow its device tensors; the
#               engine's library shares PyTorch's HIP runtime whichever is imported first,
#               tests/test_gpu_import_order.py)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    import __graft_entry__
    __graft_entry__.ensure_built()      # builds only in a tree without the library; a built one is loaded as it is


@pytest.fixture(scope="module")
def gpu_server():
    """One engine per test module: 6 GiB pool, 4 GiB LRU budget."""
    from torpor_amd.server import Server

    s = Server(mem_limit_bytes=4 << 30, pool_bytes=6 << 30)
    yield s
    s.close()
