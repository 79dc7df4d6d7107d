"""Pins the C oracle (oracle/ops_ref.c): each function against the PyTorch CPU library routine of
the same operation and against closed forms, so that a dropped term, a wrong index or a
transposed operand in the oracle fails here before it can mislead a GPU parity test."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ops as ref


def _rand(rng, *shape):
    return rng.standard_normal(shape).astype(np.float32)


def _close(a, b, tol=2e-5):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    assert a.shape == b.shape
    assert np.abs(a - b).max() <= tol * max(np.abs(b).max(), 1e-30)


@pytest.mark.parametrize("M,N,K", [(5, 7, 9), (33, 17, 64), (1, 1, 1)])
def test_gemm_vs_matmul(M, N, K):
    rng = np.random.default_rng(M)
    X, Y = _rand(rng, M, K), _rand(rng, N, K)
    want = (torch.from_numpy(X).double() @ torch.from_numpy(Y).double().T).numpy()
    _close(ref.gemm(X, Y, M, N, K, K, 1, K, 1, N).reshape(M, N), want)
    # strided views: X stored [K][M], Y stored [K][N], C with pitch N+3
    got = ref.gemm(X.T.copy(), Y.T.copy(), M, N, K, 1, M, 1, N, N + 3)
    got = np.concatenate([got, np.zeros(3, np.float32)]).reshape(M, N + 3)[:, :N]
    _close(got, want)
    # alpha / beta
    C0 = _rand(rng, M, N)
    _close(ref.gemm(X, Y, M, N, K, K, 1, K, 1, N, alpha=0.5, beta=-2.0, C_in=C0).reshape(M, N), 0.5 * want - 2.0 * C0)


@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_sgemm_colmajor_vs_numpy(ta, tb):
    rng = np.random.default_rng(ta * 2 + tb)
    m, n, k = 6, 5, 4
    A = _rand(rng, k, m) if ta else _rand(rng, m, k)       # logical op(A) is m x k
    B = _rand(rng, n, k) if tb else _rand(rng, k, n)
    opA = A.T if ta else A
    opB = B.T if tb else B
    C0 = _rand(rng, m, n)
    want = 1.5 * (opA.astype(np.float64) @ opB.astype(np.float64)) - 0.5 * C0
    # column-major storage of a (r x c) matrix is the row-major storage of its transpose
    got = ref.sgemm_colmajor(ta, tb, m, n, k, 1.5, A.T.copy(), A.shape[0], B.T.copy(), B.shape[0], -0.5,
                             C0.T.copy(), m)
    _close(got.reshape(n, m).T, want)


@pytest.mark.parametrize("k,stride,pad", [(1, 1, 0), (3, 1, 1), (3, 2, 1), (7, 2, 3), (5, 3, 0)])
def test_conv_vs_torch(k, stride, pad):
    rng = np.random.default_rng(k * 10 + stride)
    x, w = _rand(rng, 2, 5, 13, 11), _rand(rng, 6, 5, k, k)
    want = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), stride=stride, padding=pad).numpy()
    _close(ref.conv2d(x, w, (stride, stride), (pad, pad)), want)
    x_nhwc = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    _close(ref.conv2d(x_nhwc, w, (stride, stride), (pad, pad), x_nhwc=True, y_nhwc=True), want.transpose(0, 2, 3, 1))
    _close(ref.conv2d(x_nhwc, w, (stride, stride), (pad, pad), x_nhwc=True, y_nhwc=False), want)


def test_conv_delta_kernel_is_identity():
    rng = np.random.default_rng(0)
    x = _rand(rng, 1, 4, 6, 6)
    w = np.zeros((4, 4, 3, 3), np.float32)
    for c in range(4):
        w[c, c, 1, 1] = 1
    np.testing.assert_array_equal(ref.conv2d(x, w, (1, 1), (1, 1)), x)


@pytest.mark.parametrize("nhwc", [True, False])
def test_bn_vs_torch(nhwc):
    rng = np.random.default_rng(3)
    x = _rand(rng, 2, 6, 5, 4)          # NCHW
    g, b, mu = _rand(rng, 6), _rand(rng, 6), _rand(rng, 6)
    var = rng.uniform(0.2, 2, 6).astype(np.float32)
    want = F.batch_norm(torch.from_numpy(x).double(), torch.from_numpy(mu).double(), torch.from_numpy(var).double(),
                        torch.from_numpy(g).double(), torch.from_numpy(b).double(), False, 0.0, 1e-5).numpy()
    if nhwc:
        got = ref.bn(np.ascontiguousarray(x.transpose(0, 2, 3, 1)), g, b, mu, var, 1e-5, 6, nhwc=True)
        _close(got.transpose(0, 3, 1, 2), want, 1e-6)
    else:
        _close(ref.bn(x, g, b, mu, var, 1e-5, 6, hw=20, nhwc=False), want, 1e-6)
        _close(ref.bn(x, g, b, mu, var, 1e-5, 6, hw=20, nhwc=False, relu=True), np.maximum(want, 0), 1e-6)


def test_layernorm_softmax_gelu_vs_torch():
    rng = np.random.default_rng(4)
    x, r = _rand(rng, 7, 48) * 3 + 1, _rand(rng, 7, 48)
    g, b = _rand(rng, 48), _rand(rng, 48)
    want = F.layer_norm(torch.from_numpy(x + r).double(), (48,), torch.from_numpy(g).double(),
                        torch.from_numpy(b).double(), 1e-12).numpy()
    _close(ref.layernorm(x, r, g, b, 1e-12), want, 1e-6)
    y = ref.layernorm(x, None, np.ones(48, np.float32), np.zeros(48, np.float32), 1e-12).astype(np.float64)
    assert np.abs(y.mean(1)).max() < 1e-6 and np.abs(y.var(1) - 1).max() < 1e-5
    mask = np.where(rng.random((7, 48)) < 0.3, -1e9, 0).astype(np.float32)
    want = torch.softmax(torch.from_numpy(x).double() * 0.25 + torch.from_numpy(mask).double(), -1).numpy()
    got = ref.softmax(x, mask, 0.25, 1)
    _close(got, want, 1e-6)
    assert np.abs(got.astype(np.float64).sum(1) - 1).max() < 1e-6
    _close(ref.gelu(x), F.gelu(torch.from_numpy(x).double()).numpy(), 1e-6)
    assert ref.gelu(np.zeros(1, np.float32))[0] == 0


def test_depthwise_avgpool2d_activations_vs_torch():
    rng = np.random.default_rng(11)
    x, w = _rand(rng, 2, 9, 7, 8), _rand(rng, 8, 1, 3, 3)
    for stride, pad in ((1, 1), (2, 1), (1, 0)):
        want = F.conv2d(torch.from_numpy(x).double().permute(0, 3, 1, 2), torch.from_numpy(w).double(), stride=stride,
                        padding=pad, groups=8).permute(0, 2, 3, 1).numpy()
        _close(ref.depthwise_conv2d(x, w, (stride, stride), (pad, pad)), want, 1e-6)
    w5 = _rand(rng, 8, 1, 5, 5)
    want = F.conv2d(torch.from_numpy(x).double().permute(0, 3, 1, 2), torch.from_numpy(w5).double(), stride=2, padding=2,
                    groups=8).permute(0, 2, 3, 1).numpy()
    _close(ref.depthwise_conv2d(x, w5, (2, 2), (2, 2)), want, 1e-6)
    for k, stride, pad in ((2, 2, 0), (3, 1, 1), (3, 2, 1)):
        want = F.avg_pool2d(torch.from_numpy(x).double().permute(0, 3, 1, 2), k, stride, pad).permute(0, 2, 3, 1).numpy()
        _close(ref.avgpool2d(x, k, stride, pad), want, 1e-6)
    t = torch.from_numpy(x).double() * 4
    _close(ref.activation(x * 4, "relu6"), F.relu6(t).numpy(), 1e-7)
    _close(ref.activation(x * 4, "silu"), F.silu(t).numpy(), 1e-6)
    _close(ref.activation(x * 4, "sigmoid"), torch.sigmoid(t).numpy(), 1e-6)


def test_attention_vs_torch():
    """The fused-attention oracle against torch's scaled_dot_product_attention (float64), with
    and without an additive key mask, and against the closed form for identical keys (uniform
    probabilities -> the mean of V)."""
    rng = np.random.default_rng(9)
    B, S, A, dh = 2, 37, 3, 16
    q, k, v = _rand(rng, B, S, A, dh), _rand(rng, B, S, A, dh), _rand(rng, B, S, A, dh)
    mask = np.where(rng.random((B, S)) < 0.3, -1e4, 0).astype(np.float32)
    mask[:, 0] = 0
    tq, tk, tv = (torch.from_numpy(t).double().permute(0, 2, 1, 3) for t in (q, k, v))
    for m in (None, mask):
        am = None if m is None else torch.from_numpy(m).double()[:, None, None, :]
        want = F.scaled_dot_product_attention(tq, tk, tv, attn_mask=am, scale=0.25).permute(0, 2, 1, 3).numpy()
        _close(ref.attention(q, k, v, m, 0.25), want, 1e-6)
    same_k = np.broadcast_to(k[:, :1], k.shape)
    _close(ref.attention(q, same_k, v, None, 0.7), np.broadcast_to(v.mean(1, keepdims=True), v.shape), 1e-6)


@pytest.mark.parametrize("nhwc", [True, False])
def test_pool_vs_torch(nhwc):
    rng = np.random.default_rng(5)
    x = _rand(rng, 2, 3, 9, 8)
    xin = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if nhwc else x
    want = F.max_pool2d(torch.from_numpy(x), 3, 2, 1).numpy()
    got = ref.maxpool(xin, 3, 2, 1, nhwc=nhwc)
    np.testing.assert_array_equal(got.transpose(0, 3, 1, 2) if nhwc else got, want)
    _close(ref.avgpool(xin, nhwc=nhwc), x.astype(np.float64).mean((2, 3)), 1e-6)


def test_embedding_vs_torch():
    rng = np.random.default_rng(6)
    word, pos, typ = _rand(rng, 30, 8), _rand(rng, 10, 8), _rand(rng, 2, 8)
    ids = rng.integers(0, 30, (3, 5))
    tids = rng.integers(0, 2, (3, 5))
    want = (F.embedding(torch.from_numpy(ids), torch.from_numpy(word)) + torch.from_numpy(pos)[:5][None]
            + F.embedding(torch.from_numpy(tids), torch.from_numpy(typ))).numpy().reshape(15, 8)
    _close(ref.embedding(ids, tids, word, pos, typ, 5), want, 1e-6)
