"""The engine's library and PyTorch in one process, in either import order, share one HIP runtime and both see
the GPU (PyTorch is only plumbing here -- device tensors for the tests -- but a caller may well import it late)."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

ENGINE_FIRST = r"""
import sys
sys.path.insert(0, %(root)r)
from torpor_amd import _lib
from torpor_amd.server import Server
s = Server(pool_bytes=64 << 20)          # initialises the HIP runtime through the engine
assert "torch" not in sys.modules
import torch
assert torch.cuda.is_available(), "torch sees no device after the engine's library was loaded first"
x = torch.arange(8, device="cuda", dtype=torch.float32)
assert float((x * 2).sum().item()) == 56.0
s.close()
print("order ok")
"""

TORCH_FIRST = r"""
import sys
sys.path.insert(0, %(root)r)
import torch
assert torch.cuda.is_available()
x = torch.arange(8, device="cuda", dtype=torch.float32)
from torpor_amd.server import Server
s = Server(pool_bytes=64 << 20)
assert float((x * 2).sum().item()) == 56.0
s.close()
print("order ok")
"""


@pytest.mark.gpu
@pytest.mark.parametrize("script", [ENGINE_FIRST, TORCH_FIRST], ids=["engine-first", "torch-first"])
def test_engine_and_torch_share_the_gpu_in_either_import_order(script):
    r = subprocess.run([sys.executable, "-c", script % {"root": ROOT}], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "order ok" in r.stdout, (r.stdout[-1000:], r.stderr[-3000:])


def test_one_hip_runtime_is_mapped_when_the_engine_library_is_loaded_before_torch():
    """No GPU needed: after `torpor_amd._lib.lib()` and then `import torch` the process maps one libamdhip64."""
    code = r"""
import re, sys
sys.path.insert(0, %(root)r)
from torpor_amd import _lib
_lib.lib()
assert "torch" not in sys.modules
import torch
libs = sorted(set(re.findall(r"/\S*libamdhip64\S*", open("/proc/self/maps").read())))
assert len(libs) == 1, libs
print("one runtime")
""" % {"root": ROOT}
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "one runtime" in r.stdout, (r.stdout[-1000:], r.stderr[-3000:])
