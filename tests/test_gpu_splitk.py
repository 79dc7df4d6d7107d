"""A K range split over workgroups is summed inside the launch by the workgroup that finishes a tile last
(partial sums and ticket counters move with agent-scope accesses between the eight L2s).  Its results must
equal, bit for bit, those of the two-launch form (partial sums to memory, a reduction kernel), on every
call: the same workspace is reused with new data, so a stale cached partial sum would show."""
import os
import subprocess
import sys
import tempfile

import numpy as np
import pytest

from tests.harness import OpSession, assert_close
from torpor_amd.server import ACT_RELU, Server

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

GEMMS = [(128, 768, 3072), (196, 256, 1024), (9, 1000, 2048), (49, 512, 2048), (100, 37, 52 * 16), (128, 768, 3072)]
CONVS = [(1, 14, 14, 256, 256, 1), (8, 14, 14, 256, 256, 1), (1, 7, 7, 512, 512, 1), (1, 28, 28, 256, 256, 2),
         (2, 9, 9, 24, 40, 1)]
ROUNDS = 3


def _run_cases():
    """Every case `ROUNDS` times with fresh data, interleaved, on one engine; returns the outputs."""
    out = {}
    with Server(mem_limit_bytes=1 << 30, pool_bytes=2 << 30) as s:
        for rnd in range(ROUNDS):
            for ci, (M, N, K) in enumerate(GEMMS):
                rng = np.random.default_rng(1000 * rnd + ci)
                X = rng.standard_normal((M, K)).astype(np.float32)
                W = rng.standard_normal((N, K)).astype(np.float32)
                b = rng.standard_normal(N).astype(np.float32)
                with OpSession(s, [W, b]) as t:
                    x = t.act(X)
                    c = t.empty(M * N * 4)
                    t.s.gemm(t.fid, x, t.w[0], c, M, N, K, xs_r=K, ys_c=K, ldc=N, bias=t.w[1], act=ACT_RELU)
                    out[f"gemm{ci}_r{rnd}"] = t.read(c, (M, N))
                    out[f"gemm{ci}_r{rnd}_kernel"] = np.frombuffer(t.s.last_kernel().encode(), np.uint8)
            for ci, (n, h, w, cin, cout, stride) in enumerate(CONVS):
                rng = np.random.default_rng(5000 + 1000 * rnd + ci)
                X = rng.standard_normal((n, h, w, cin)).astype(np.float32)
                Wt = (rng.standard_normal((cout, cin, 3, 3)) / np.sqrt(9 * cin)).astype(np.float32)
                ho = (h + 2 - 3) // stride + 1
                with OpSession(s, [Wt]) as t:
                    x = t.act(X)
                    y = t.empty(n * ho * ho * cout * 4)
                    t.s.conv(t.fid, x, t.w[0], y, n, h, w, cin, cout, 3, 3, stride=stride, pad=1)
                    out[f"conv{ci}_r{rnd}"] = t.read(y, (n, ho, ho, cout))
                    out[f"conv{ci}_r{rnd}_kernel"] = np.frombuffer(t.s.last_kernel().encode(), np.uint8)
    return out


def _dump(path):
    np.savez(path, **_run_cases())


def _in_subprocess(mode, path):
    env = dict(os.environ, TORPOR_SPLITK_FUSED=mode)
    r = subprocess.run([sys.executable, "-c", f"import sys; sys.path.insert(0, {ROOT!r}); "
                        f"from tests.test_gpu_splitk import _dump; _dump({path!r})"],
                       env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr[-3000:]
    return np.load(path)


def test_in_launch_summation_equals_the_two_launch_form_bit_for_bit(monkeypatch):
    # the direct kernels are meant: the Winograd path (which the 1.85 GFLOP convolution would take) has no
    # two-launch form to compare with (the subprocesses inherit the setting)
    monkeypatch.setenv("TORPOR_WINOGRAD", "0")
    got = _run_cases()   # the library's own choice: in-launch up to 8 slots, a reduction launch above
    # the first GEMM and the first convolution of each round against float64 (the values are right at all)
    for rnd in range(ROUNDS):
        M, N, K = GEMMS[0]
        rng = np.random.default_rng(1000 * rnd)
        X = rng.standard_normal((M, K)).astype(np.float32)
        W = rng.standard_normal((N, K)).astype(np.float32)
        b = rng.standard_normal(N).astype(np.float32)
        want = np.maximum(X.astype(np.float64) @ W.astype(np.float64).T + b, 0)
        assert_close(got[f"gemm0_r{rnd}"], want, 2e-5, f"gemm round {rnd}")
    with tempfile.TemporaryDirectory() as d:
        ref = _in_subprocess("0", os.path.join(d, "two_launch.npz"))      # always a reduction launch
        every = _in_subprocess("2", os.path.join(d, "in_launch.npz"))     # always summed inside the launch
        assert set(ref.files) == set(got) == set(every.files)
        split_seen = 0
        for k in sorted(got):
            assert np.array_equal(got[k], ref[k]), k
            assert np.array_equal(every[k], ref[k]), k
            if k.endswith("_kernel"):
                split_seen += 1
    assert split_seen == ROUNDS * (len(GEMMS) + len(CONVS))
