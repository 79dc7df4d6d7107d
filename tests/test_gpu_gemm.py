"""GEMM kernels vs the fp64-accumulating C oracle, through the C-ABI (reference call sites
cublasSgemm / cublasSgemmStridedBatched, include/server/cuda_server.hpp:502-550)."""
import numpy as np
import pytest

from oracle import ops as ref
from tests.harness import OpSession, assert_close
from torpor_amd.server import ACT_GELU, ACT_NONE, ACT_RELU, ACT_TANH

pytestmark = pytest.mark.gpu
RTOL = 2e-5  # fp32 accumulation over K <= 4608 against fp64; stated bar for logits is 1e-3


def _rand(rng, *shape):
    return rng.standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("M,N,K,kernel", [
    (128, 768, 768, "gemm_fast_32x32_kc"),      # BERT-base projection: 24 64x64 tiles -> 96 32x32 tiles
    (128, 3072, 768, "gemm_fast_32x32_kc"),     # 96 64x64 tiles -> 384 32x32 tiles, K split in the workgroup
    (1536, 1024, 1024, "gemm_fast_64x32_kc"),   # BERT-large projection: 384 64x64 tiles = 1.5 per CU -> 64x32
    (1536, 1024, 4096, "gemm_fast_64x64_kc"),   # BERT-large FFN down-projection: long K, two K halves per 64x64 tile summed in the launch
    (4096, 2048, 160, "gemm_fast_64x64_kc"),    # K % 64 != 0: predicated kernel
    (1, 1000, 2048, "gemv_rows_kc"),            # ResNet classifier, batch 1: a matrix-vector product, one wavefront per column
    (9, 1000, 2048, "gemm_fast_32x32_kc"),      # one row more than the matrix-vector path takes: 32 small tiles, K split over 8 workgroups each
    (1568, 256, 1024, "gemm_fast_32x32_kc"),    # ResNet-152 batch 8 layer3 1x1: 100 64x64 tiles -> 32x32, K split in the workgroup
    (49, 512, 2048, "gemm_fast_32x32_kc"),      # ragged M (ResNet-50 batch 1, 7x7 pixels)
    (100, 37, 52, "gemm_fast_64x64_kc"),        # ragged N, K % 32 != 0
    (33, 65, 7, "gemm_generic_64x64"),          # K % 4 != 0 -> scalar path
])
def test_gemm_tn(gpu_server, M, N, K, kernel):
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    X, W, b = _rand(rng, M, max(K, 1))[:, :K], _rand(rng, N, max(K, 1))[:, :K], _rand(rng, N)
    X, W = np.ascontiguousarray(X), np.ascontiguousarray(W)
    with OpSession(gpu_server, [W if K else np.zeros(1, np.float32), b]) as t:
        x = t.act(X if K else np.zeros(1, np.float32))
        c = t.empty(M * N * 4)
        t.s.gemm(t.fid, x, t.w[0], c, M, N, K, xs_r=max(K, 1), ys_c=max(K, 1), ldc=N, bias=t.w[1])
        if kernel:
            assert t.s.last_kernel().startswith(kernel), t.s.last_kernel()
        got = t.read(c, (M, N))
    if M * N * K > 5e7:   # too slow for the triple loop: fp64 BLAS matmul instead
        want = X.astype(np.float64) @ W.astype(np.float64).T + b
    else:
        want = ref.gemm(X, W, M, N, K, max(K, 1), 1, max(K, 1), 1, N).reshape(M, N) + b
    assert_close(got, want, RTOL, f"gemm {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [
    (1, 20, 480),        # squeeze-and-excitation, first layer (EfficientNet-B0)
    (1, 480, 20),        # ... second layer: K shorter than one wavefront step
    (1, 1001, 1028),     # odd column count, K not a multiple of the 256-float step
    (2, 768, 768),       # MR = 2
    (3, 33, 4),          # MR = 4 with one row unused, a single 128-bit step
    (5, 130, 2052),      # MR = 8 with three rows unused
    (8, 1000, 2048),     # ResNet-152 batch 8 classifier
    (1, 4096, 25088),    # VGG-16 first fully connected layer: 411 MB of weights read once
])
def test_gemm_of_few_rows_runs_as_matrix_vector_products(gpu_server, M, N, K):
    rng = np.random.default_rng(M * 11 + N * 5 + K)
    X, W, b, R = _rand(rng, M, K), _rand(rng, N, K), _rand(rng, N), _rand(rng, M, N)
    with OpSession(gpu_server, [W, b]) as t:
        x, r = t.act(X), t.act(R)
        c = t.empty(M * N * 4)
        t.s.gemm(t.fid, x, t.w[0], c, M, N, K, xs_r=K, ys_c=K, ldc=N, bias=t.w[1], residual=r, act=ACT_RELU)
        assert t.s.last_kernel() == "gemv_rows_kc", t.s.last_kernel()
        got = t.read(c, (M, N))
        t.s.gemm(t.fid, x, t.w[0], c, M, N, K, xs_r=K, ys_c=K, ldc=N, bias=t.w[1], residual=r, act=ACT_RELU)
        again = t.read(c, (M, N))
    if M * N * K > 5e7:   # too slow for the oracle's triple loop: fp64 BLAS matmul instead
        want = np.maximum(X.astype(np.float64) @ W.astype(np.float64).T + b + R, 0)
    else:
        want = np.maximum(ref.gemm(X, W, M, N, K, K, 1, K, 1, N).reshape(M, N).astype(np.float64) + b + R, 0)
    assert_close(got, want, RTOL, f"gemv {M}x{N}x{K}")
    assert np.array_equal(got, again), "a repeated launch must give the same bits"


def test_matrix_vector_path_applies_alpha_beta_and_batch_norm(gpu_server):
    rng = np.random.default_rng(77)
    M, N, K = 4, 96, 260
    X, W, C0 = _rand(rng, M, K), _rand(rng, N, K), _rand(rng, M, N)
    g, b, mu = _rand(rng, N), _rand(rng, N), _rand(rng, N)
    var = rng.uniform(0.5, 2.0, N).astype(np.float32)
    with OpSession(gpu_server, [W, g, b, mu, var]) as t:
        x, c = t.act(X), t.act(C0)
        t.s.gemm(t.fid, x, t.w[0], c, M, N, K, xs_r=K, ys_c=K, ldc=N, alpha=0.5, beta=2.0, bn=tuple(t.w[1:5]),
                 bn_eps=1e-5, act=ACT_TANH)
        assert t.s.last_kernel() == "gemv_rows_kc", t.s.last_kernel()
        got = t.read(c, (M, N))
    z = 0.5 * ref.gemm(X, W, M, N, K, K, 1, K, 1, N).reshape(M, N).astype(np.float64) + 2.0 * C0
    want = np.tanh((z - mu) / np.sqrt(var.astype(np.float64) + 1e-5) * g + b)
    assert_close(got, want, 5e-5, "gemv alpha/beta/bn/tanh")


@pytest.mark.parametrize("act", [ACT_NONE, ACT_RELU, ACT_GELU, ACT_TANH])
def test_gemm_epilogue(gpu_server, act):
    rng = np.random.default_rng(act)
    M, N, K = 70, 96, 128
    X, W, b, R, C0 = _rand(rng, M, K), _rand(rng, N, K), _rand(rng, N), _rand(rng, M, N), _rand(rng, M, N)
    with OpSession(gpu_server, [W, b]) as t:
        x, r, c = t.act(X), t.act(R), t.act(C0)
        t.s.gemm(t.fid, x, t.w[0], c, M, N, K, xs_r=K, ys_c=K, ldc=N, bias=t.w[1], alpha=0.5, beta=2.0,
                 residual=r, act=act)
        got = t.read(c, (M, N))
    z = 0.5 * ref.gemm(X, W, M, N, K, K, 1, K, 1, N).reshape(M, N).astype(np.float64) + 2.0 * C0 + b + R
    if act == ACT_RELU:
        z = np.maximum(z, 0)
    elif act == ACT_GELU:
        z = ref.gelu(z.astype(np.float32)).astype(np.float64)
    elif act == ACT_TANH:
        z = np.tanh(z)
    assert_close(got, z, 5e-5, f"epilogue act={act}")


def test_gemm_bn_epilogue(gpu_server):
    rng = np.random.default_rng(5)
    M, N, K = 64, 80, 64
    X, W = _rand(rng, M, K), _rand(rng, N, K)
    g, b, mu = _rand(rng, N), _rand(rng, N), _rand(rng, N)
    var = rng.uniform(0.5, 2.0, N).astype(np.float32)
    with OpSession(gpu_server, [W, g, b, mu, var]) as t:
        x = t.act(X)
        c = t.empty(M * N * 4)
        t.s.gemm(t.fid, x, t.w[0], c, M, N, K, xs_r=K, ys_c=K, ldc=N, bn=tuple(t.w[1:5]), bn_eps=1e-5, act=ACT_RELU)
        got = t.read(c, (M, N))
    z = ref.gemm(X, W, M, N, K, K, 1, K, 1, N).reshape(M, N)
    want = ref.bn(z, g, b, mu, var, 1e-5, N, nhwc=True, relu=True)
    assert_close(got, want, 5e-5, "gemm+bn+relu")


@pytest.mark.parametrize("B,A,S,dh", [(1, 12, 128, 64), (2, 4, 96, 64), (1, 3, 50, 24)])
def test_attention_gemms(gpu_server, B, A, S, dh):
    """Head-strided batched products read in place from [tokens, hidden] projections:
    scores = Q.K^T (both K-contiguous) and ctx = P.V (V c-contiguous)."""
    rng = np.random.default_rng(B + A + S)
    H = A * dh
    Q, Kx, V = _rand(rng, B * S, H), _rand(rng, B * S, H), _rand(rng, B * S, H)
    with OpSession(gpu_server, [np.zeros(4, np.float32)]) as t:
        q, k, v = t.act(Q), t.act(Kx), t.act(V)
        sc = t.empty(B * A * S * S * 4)
        t.s.gemm(t.fid, q, k, sc, S, S, dh, xs_r=H, ys_c=H, ldc=S, nb0=B, nb1=A, xb0=S * H, xb1=dh, yb0=S * H,
                 yb1=dh, cb0=A * S * S, cb1=S * S)
        k1 = t.s.last_kernel()
        scores = t.read(sc, (B, A, S, S))
        ctx = t.empty(B * S * H * 4)
        t.s.gemm(t.fid, sc, v, ctx, S, dh, S, xs_r=S, ys_c=1, ys_k=H, ldc=H, nb0=B, nb1=A, xb0=A * S * S,
                 xb1=S * S, yb0=S * H, yb1=dh, cb0=S * H, cb1=dh)
        k2 = t.s.last_kernel()
        got_ctx = t.read(ctx, (B, S, A, dh))
    if dh % 4 == 0 and S % 4 == 0:
        assert "_kc" in k1 and "_cc" in k2, (k1, k2)
    Qh = Q.reshape(B, S, A, dh).transpose(0, 2, 1, 3).astype(np.float64)
    Kh = Kx.reshape(B, S, A, dh).transpose(0, 2, 1, 3).astype(np.float64)
    Vh = V.reshape(B, S, A, dh).transpose(0, 2, 1, 3).astype(np.float64)
    want = Qh @ Kh.transpose(0, 1, 3, 2)
    assert_close(scores, want, RTOL, "scores")
    want_ctx = (scores.astype(np.float64) @ Vh).transpose(0, 2, 1, 3)
    assert_close(got_ctx, want_ctx, RTOL, "ctx")


@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_sgemm_colmajor(gpu_server, ta, tb):
    """cublasSgemm argument convention, all four transpose combinations, alpha/beta."""
    rng = np.random.default_rng(ta * 2 + tb)
    m, n, k = 45, 52, 36
    lda = (m if not ta else k) + 3
    ldb = (k if not tb else n) + 1
    ldc = m + 2
    A = _rand(rng, lda * (k if not ta else m))
    Bm = _rand(rng, ldb * (n if not tb else k))
    C0 = _rand(rng, ldc * n)
    with OpSession(gpu_server, [A]) as t:
        b, c = t.act(Bm), t.act(C0)
        t.s.sgemm(t.fid, ta, tb, m, n, k, 1.5, t.w[0], lda, b, ldb, -0.5, c, ldc)
        got = t.read(c, (ldc * n,))
    want = ref.sgemm_colmajor(ta, tb, m, n, k, 1.5, A, lda, Bm, ldb, -0.5, C0, ldc)
    assert_close(got, want, RTOL, f"sgemm ta={ta} tb={tb}")


def test_gemm_rejects_out_of_bounds(gpu_server):
    from torpor_amd._lib import TorporError
    with OpSession(gpu_server, [np.zeros((8, 8), np.float32)]) as t:
        x = t.act(np.zeros((4, 8), np.float32))
        c = t.empty(4 * 8 * 4)
        with pytest.raises(TorporError):
            t.s.gemm(t.fid, x, t.w[0], c, 5, 8, 8, xs_r=8, ys_c=8, ldc=8)   # X has 4 rows
        with pytest.raises(TorporError):
            t.s.gemm(t.fid, x, t.w[0], c, 4, 9, 8, xs_r=8, ys_c=8, ldc=9)   # W has 8 rows
        with pytest.raises(TorporError):
            t.s.stream_synchronize(t.fid)   # the refused ops are also reported (once) at the next sync
        t.s.gemm(t.fid, x, t.w[0], c, 4, 8, 8, xs_r=8, ys_c=8, ldc=8)


@pytest.mark.parametrize("cfg,name", [(0, "128x128"), (1, "128x64"), (2, "64x64"), (3, "64x32"), (4, "32x32")])
def test_forced_tile_configs(cfg, name):
    """Every tile shape of the fast kernel (TORPOR_GEMM_CFG forces one; read once per process,
    hence the subprocess): ragged and exact shapes, predicated and branch-free variants."""
    import os
    import subprocess
    import sys
    code = r'''
import numpy as np, sys
from torpor_amd.server import Server
from tests.harness import OpSession, assert_close
rng = np.random.default_rng(0)
with Server(mem_limit_bytes=1 << 30, pool_bytes=2 << 30) as s:
    for (M, N, K) in [(200, 136, 128), (257, 130, 100), (64, 64, 64), (300, 520, 192), (257, 130, 256), (300, 100, 384)]:
        X = rng.standard_normal((M, K)).astype(np.float32)
        W = rng.standard_normal((N, K)).astype(np.float32)
        V = rng.standard_normal((K, N)).astype(np.float32)
        with OpSession(s, [W]) as t:
            x, v = t.act(X), t.act(V)
            c = t.empty(M * N * 4)
            s.gemm(t.fid, x, t.w[0], c, M, N, K, xs_r=K, ys_c=K, ldc=N)
            # the tiles that split K over wavefronts exist for whole 64-wide K-blocks only: pairs of them for
            # 64x32 (K % 128 == 0), any number for 32x32 (K % 64 == 0)
            need = {"64x32": 128, "32x32": 64}.get(sys.argv[1], 1)
            want = sys.argv[1] if (K % need == 0 and (need == 1 or K >= 128)) else "64x64"
            assert want in s.last_kernel(), s.last_kernel()
            assert_close(t.read(c, (M, N)), X.astype(np.float64) @ W.astype(np.float64).T, 2e-5, "kc")
            s.gemm(t.fid, x, v, c, M, N, K, xs_r=K, ys_c=1, ys_k=N, ldc=N)
            assert_close(t.read(c, (M, N)), X.astype(np.float64) @ V.astype(np.float64), 2e-5, "cc")
print("ok")
'''
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, TORPOR_GEMM_CFG=str(cfg), PYTHONPATH=root)
    r = subprocess.run([sys.executable, "-c", code, name], env=env, cwd=root, capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0 and "ok" in r.stdout, r.stdout + r.stderr
