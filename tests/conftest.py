import os
import sys

import pytest
import torch  # noqa: F401  (first: PyTorch ships its own HIP runtime, and in a process that uses both that one
#               has to be loaded before the engine's library initialises the system's; the other order
#               leaves torch.cuda without a device)

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
