"""tp_gemm_ln: a LayerNorm between two GEMMs without a launch of its own.  The first GEMM stores per-row statistics
of its output (mean and squared deviations per block of 32 columns), the second normalises its X operand from them
while loading it and writes the normalised rows out.  Checked against the fp64 oracle chain GEMM -> LayerNorm -> GEMM
(oracle/ops.py; the reference forwards these as cublasSgemm, a LayerNorm launch and cublasSgemm:
include/server/cuda_server.hpp:502-522,1226-1310), over the shapes of the BERT layers and over shapes for which the
kernels have no fused variant (the same arithmetic then runs as launches of its own)."""
import numpy as np
import pytest

from oracle import ops as ref
from tests.harness import OpSession, assert_close
from torpor_amd.server import ACT_GELU, ACT_NONE, TorporError

pytestmark = pytest.mark.gpu
EPS = 1e-12


def _rand(rng, *shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(np.float32)


def _block_stats(c):
    """(mean, sum of squared deviations) per row and block of 32 columns, in float64."""
    m, n = c.shape
    b = c.astype(np.float64).reshape(m, n // 32, 32)
    mean = b.mean(axis=2)
    return np.stack([mean, ((b - mean[..., None]) ** 2).sum(axis=2)], axis=2)


# M, H (width of the normalised rows), N2 (columns of the consuming GEMM), K1 (depth of the producing GEMM)
CASES = [
    (128, 768, 2304, 768),      # BERT-base: attention output -> LayerNorm -> ... (32x32 tiles, K split inside the launch)
    (128, 768, 3072, 3072),     # BERT-base: FFN down -> LayerNorm -> FFN up of the shapes' sizes
    (1536, 1024, 3072, 1024),   # BERT-large: 64x32 producer, 64x64 consumer with two LDS stages
    (1536, 1024, 4096, 4096),   # BERT-large: FFN down (K 4096) -> FFN up (one LDS stage)
    (512, 1024, 3072, 1024),    # question answering at sequence 512: 64x32 consumer
    (100, 256, 160, 96),        # ragged rows, a producer whose K is no multiple of 64 (predicated kernel)
    (37, 96, 72, 40),           # N not a multiple of the tile: statistics by the fallback kernel; consumer falls back too
    (9, 64, 8, 2048),           # deep split of the producer's K (a reduction launch): fallback statistics
]


@pytest.mark.parametrize("M,H,N2,K1", CASES)
def test_gemm_layernorm_gemm(gpu_server, M, H, N2, K1):
    rng = np.random.default_rng(M + H + N2 + K1)
    x = _rand(rng, M, K1)
    w1 = _rand(rng, H, K1, scale=1.0 / np.sqrt(K1))
    b1 = _rand(rng, H)
    res = _rand(rng, M, H) + np.float32(0.5)          # a residual with a mean: the statistics must not assume zero mean
    gamma = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    beta = _rand(rng, H, scale=0.1)
    w2 = _rand(rng, N2, H, scale=1.0 / np.sqrt(H))
    b2 = _rand(rng, N2)
    with OpSession(gpu_server, [w1, b1, gamma, beta, w2, b2]) as t:
        xv, rv = t.act(x), t.act(res)
        pre = t.empty(M * H * 4)
        stats = t.empty(M * (H // 32) * 2 * 4)
        normed = t.empty(M * H * 4)
        out = t.empty(M * N2 * 4)
        t.s.gemm(t.fid, xv, t.w[0], pre, M, H, K1, xs_r=K1, ys_c=K1, ldc=H, bias=t.w[1], residual=rv, ln_stats_out=stats)
        k1 = t.s.last_kernel()
        t.s.gemm(t.fid, pre, t.w[4], out, M, N2, H, xs_r=H, ys_c=H, ldc=N2, bias=t.w[5], act=ACT_GELU,
                 ln_a=(stats, t.w[2], t.w[3], normed, EPS))
        k2 = t.s.last_kernel()
        print(f"{M}x{H}x{K1} {k1} -> {M}x{N2}x{H} {k2}", flush=True)
        got_pre = t.read(pre, (M, H))
        got_stats = t.read(stats, (M, H // 32, 2))
        got_normed = t.read(normed, (M, H))
        got_out = t.read(out, (M, N2))
        # the same pair without the fusion: a LayerNorm launch of its own between two plain GEMMs
        pre2, normed2, out2 = t.empty(M * H * 4), t.empty(M * H * 4), t.empty(M * N2 * 4)
        t.s.gemm(t.fid, xv, t.w[0], pre2, M, H, K1, xs_r=K1, ys_c=K1, ldc=H, bias=t.w[1], residual=rv)
        t.s.launch(t.fid, 7, [pre2, 0, t.w[2], t.w[3], normed2], [M, H], [EPS])
        t.s.gemm(t.fid, normed2, t.w[4], out2, M, N2, H, xs_r=H, ys_c=H, ldc=N2, bias=t.w[5], act=ACT_GELU)
        plain_pre, plain_out = t.read(pre2, (M, H)), t.read(out2, (M, N2))
    want_pre = ref.gemm(x, w1, M, H, K1, K1, 1, K1, 1, H).reshape(M, H).astype(np.float64) + b1 + res
    assert_close(got_pre, want_pre, 3e-5, "producer output")
    assert np.array_equal(got_pre, plain_pre), "the statistics must not change what the producer writes"
    want_stats = _block_stats(got_pre)
    assert_close(got_stats[..., 0], want_stats[..., 0], 1e-5, "block means")
    assert_close(got_stats[..., 1], want_stats[..., 1], 1e-4, "block squared deviations")
    want_normed = ref.layernorm(got_pre, None, gamma, beta, EPS)
    assert_close(got_normed, want_normed, 2e-5, "normalised rows")
    want_out = ref.gelu((ref.gemm(want_normed, w2, M, N2, H, H, 1, H, 1, N2).reshape(M, N2).astype(np.float64) + b2).astype(np.float32))
    assert_close(got_out, want_out, 5e-5, "consumer output")
    assert_close(got_out, plain_out, 5e-5, "fused against unfused")


def test_gemm_ln_refuses_what_it_cannot_mean(gpu_server):
    rng = np.random.default_rng(3)
    M, H = 16, 64
    w = _rand(rng, H, H)
    g = np.ones(H, np.float32)
    with OpSession(gpu_server, [w, g]) as t:
        xv = t.act(_rand(rng, M, H))
        c = t.empty(M * H * 4)
        stats = t.empty(M * 2 * 2 * 4)
        small = t.empty(16)
        with pytest.raises(TorporError):    # statistics of an activated output
            t.s.gemm(t.fid, xv, t.w[0], c, M, H, H, xs_r=H, ys_c=H, ldc=H, act=ACT_GELU, ln_stats_out=stats)
        with pytest.raises(TorporError):    # statistics buffer too small for [M][H/32][2]
            t.s.gemm(t.fid, xv, t.w[0], c, M, H, H, xs_r=H, ys_c=H, ldc=H, ln_stats_out=small)
        with pytest.raises(TorporError):    # 40 columns: no whole blocks of 32
            t.s.gemm(t.fid, xv, t.w[0], c, M, 40, H, xs_r=H, ys_c=H, ldc=40, ln_stats_out=stats)
        with pytest.raises(TorporError):    # normalised rows have nowhere to go
            t.s.gemm(t.fid, xv, t.w[0], c, M, H, H, xs_r=H, ys_c=H, ldc=H, ln_a=(stats, t.w[1], t.w[1], 0, EPS))
        with pytest.raises(TorporError):    # X is not dense
            t.s.gemm(t.fid, xv, t.w[0], c, M // 2, H, H, xs_r=2 * H, ys_c=H, ldc=H, ln_a=(stats, t.w[1], t.w[1], c, EPS))
        with pytest.raises(TorporError):    # batched
            t.s.gemm(t.fid, xv, t.w[0], c, M // 2, H, H, xs_r=H, ys_c=H, ldc=H, nb0=2, xb0=M // 2 * H, cb0=M // 2 * H,
                     ln_stats_out=stats)
        with pytest.raises(TorporError):
            t.s.stream_synchronize(t.fid)
        t.s.gemm(t.fid, xv, t.w[0], c, M, H, H, xs_r=H, ys_c=H, ldc=H, ln_stats_out=stats)
