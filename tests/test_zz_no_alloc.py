"""tp_gemm_noalloc (raw device addresses, caller's stream, fixed scratch array, no allocation) against
tp_gemm on the same inputs: bit-identical, on two calls in a row, the second with a smaller input, so
that the second call runs over the partial sums the first one left in the shared scratch array."""
import numpy as np
import pytest
import torch  # before anything initialises the system's HIP runtime: see tests/conftest.py

from tests.harness import OpSession
from torpor_amd import _lib
from torpor_amd.server import ACT_RELU, Server, gemm_noalloc

pytestmark = pytest.mark.gpu

TP_ESCRATCH = -75
SCRATCH_BYTES = 16 << 20


def _through_engine(server, X, W, b, M, N, K, act):
    with OpSession(server, [W, b]) as t:
        x = t.act(X)
        c = t.empty(M * N * 4)
        t.s.gemm(t.fid, x, t.w[0], c, M, N, K, xs_r=K, ys_c=K, ldc=N, bias=t.w[1], act=act)
        kernel = t.s.last_kernel()
        return t.read(c, (M, N)), kernel


def _no_alloc(torch, X, W, b, M, N, K, act, stream):
    dx, dw, db = (torch.from_numpy(a).cuda() for a in (X, W, b))
    dc = torch.full((M, N), float("nan"), device="cuda")
    torch.cuda.synchronize()
    # free bytes of the device as the runtime reports them (hipMemGetInfo): this sees an allocation made by any
    # library in the process, which the framework's own counter of its caching allocator would not
    before_free = torch.cuda.mem_get_info()[0]
    before = torch.cuda.memory_allocated()
    r = gemm_noalloc(dx.data_ptr(), dw.data_ptr(), dc.data_ptr(), M, N, K, xs_r=K, ys_c=K, ldc=N, bias=db.data_ptr(),
                     act=act, stream=stream.cuda_stream)
    assert r == 0, _lib.lib().tp_strerror(r)
    stream.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == before_free, "the call allocated or freed device memory"
    return dc.cpu().numpy()


def _first_call_on_this_device(torch, stream):
    """The first call on a device looks up the device's copy of the scratch array (which may load the library's
    code object and, with it, the array itself): documented to happen outside the stretch in which nothing may be
    allocated.  A small unsplit GEMM does it."""
    a = torch.ones((32, 32), device="cuda")
    c = torch.empty((32, 32), device="cuda")
    r = gemm_noalloc(a.data_ptr(), a.data_ptr(), c.data_ptr(), 32, 32, 32, xs_r=32, ys_c=32, ldc=32, stream=stream.cuda_stream)
    assert r == 0, _lib.lib().tp_strerror(r)
    stream.synchronize()
    assert float(c.min()) == float(c.max()) == 32.0


def test_no_alloc_gemm_matches_tp_gemm_twice_in_a_row():
    torch.cuda.set_device(0)
    stream = torch.cuda.Stream()
    rng = np.random.default_rng(11)
    # every shape splits K over workgroups (few output tiles, long K): the scratch array is used -- by 32x32
    # tiles whose slots are summed inside the launch, and (K not a multiple of 128) by 64x64 tiles
    shapes = [(128, 768, 3072, ACT_RELU), (96, 200, 1056, 0), (9, 1000, 2048, 0), (64, 256, 1024, 0)]
    cases = []
    for M, N, K, act in shapes:
        X = rng.standard_normal((M, K)).astype(np.float32)
        W = rng.standard_normal((N, K)).astype(np.float32)
        b = rng.standard_normal(N).astype(np.float32)
        cases.append((X, W, b, M, N, K, act))
    with Server(mem_limit_bytes=1 << 30, pool_bytes=2 << 30) as s:
        want = [_through_engine(s, *c) for c in cases]
    assert any("64x64" in k for _, k in want) and any("32x32" in k for _, k in want), [k for _, k in want]
    _first_call_on_this_device(torch, stream)
    for c, (ref, kernel) in zip(cases, want):   # largest first: later calls see stale partial sums
        print("case", c[3:], kernel, flush=True)
        got = _no_alloc(torch, *c, stream)
        assert np.array_equal(got, ref), (c[3:], kernel, float(np.abs(got - ref).max()))


_CHILD = r"""
import sys, torch
sys.path.insert(0, sys.argv[1])
from torpor_amd.server import gemm_noalloc
torch.cuda.set_device(0)
M, N, K = 960, 1024, 8224
x = torch.zeros((M, K), device="cuda"); w = torch.zeros((N, K), device="cuda"); c = torch.zeros((M, N), device="cuda")
r = gemm_noalloc(x.data_ptr(), w.data_ptr(), c.data_ptr(), M, N, K, xs_r=K, ys_c=K, ldc=N)
torch.cuda.synchronize()
print("status", r)
"""


def test_no_alloc_gemm_refuses_what_does_not_fit_or_is_malformed():
    import os
    import subprocess
    import sys

    torch.cuda.set_device(0)
    x = torch.zeros((8, 8), device="cuda")
    w = torch.zeros((8, 8), device="cuda")
    c = torch.zeros((8, 8), device="cuda")
    assert gemm_noalloc(0, w.data_ptr(), c.data_ptr(), 4, 4, 4, xs_r=4, ys_c=4, ldc=4) == -22      # null operand
    assert gemm_noalloc(x.data_ptr(), w.data_ptr(), c.data_ptr(), 4, 8, 4, xs_r=4, ys_c=4, ldc=4) == -22   # ldc < n
    assert gemm_noalloc(x.data_ptr(), w.data_ptr(), c.data_ptr(), 0, 8, 4, xs_r=4, ys_c=4, ldc=8) == -22   # m < 1
    torch.cuda.synchronize()
    # The launcher's own rule never splits K so far that the partial sums outgrow the fixed array (at most
    # about 12 MiB of its 16); the debugging switch that forces a split count does: 32 x 960 x 1024 x 4 B.
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, TORPOR_SPLITS="32")
    out = subprocess.run([sys.executable, "-c", _CHILD, root], env=env, capture_output=True, text=True, timeout=110)
    assert out.returncode == 0, out.stderr[-2000:]
    assert f"status {TP_ESCRATCH}" in out.stdout, out.stdout
