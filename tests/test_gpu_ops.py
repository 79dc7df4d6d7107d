"""HBM-bound operators vs the C oracle, through the C-ABI (reference call sites
cudnnBatchNormalizationForwardInference, include/server/cuda_server.hpp:737-771, and libtorch
kernels launched through cudaLaunchKernel, include/server/cuda_server.hpp:1226-1310)."""
import numpy as np
import pytest

from oracle import ops as ref
from tests.harness import OpSession, assert_close
from torpor_amd.server import (NCHW, NHWC, OP_ADD, OP_ATTENTION, OP_AVGPOOL, OP_BIAS_ACT, OP_EMBEDDING, OP_FILL, OP_GELU,
                               OP_LAYERNORM, OP_MAXPOOL, OP_NCHW_TO_NHWC, OP_NHWC_TO_NCHW, OP_RELU, OP_SOFTMAX,
                               OP_SUM, OP_AVGPOOL2D, OP_COPY2D, OP_SCALE_CHANNELS, ACT_RELU, ACT_RELU6, ACT_SILU, ACT_SIGMOID, TorporError)

pytestmark = pytest.mark.gpu


def _rand(rng, *shape):
    return rng.standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("layout,C,relu", [(NHWC, 64, True), (NHWC, 7, False), (NCHW, 5, True)])
def test_bn_inference(gpu_server, layout, C, relu):
    rng = np.random.default_rng(C)
    N, H, W = 2, 9, 11
    x = _rand(rng, N, H, W, C) if layout == NHWC else _rand(rng, N, C, H, W)
    g, b, mu = _rand(rng, C), _rand(rng, C), _rand(rng, C)
    var = rng.uniform(0.1, 3.0, C).astype(np.float32)
    with OpSession(gpu_server, [g, b, mu, var]) as t:
        xv = t.act(x)
        yv = t.empty(x.nbytes)
        t.s.bn(t.fid, xv, yv, *t.w[:4], 1e-5, N * H * W, C, hw=H * W, layout=layout, relu=relu)
        got = t.read(yv, x.shape)
    want = ref.bn(x, g, b, mu, var, 1e-5, C, hw=H * W, nhwc=(layout == NHWC), relu=relu)
    assert_close(got, want, 1e-6, "bn")


def test_bn_identity(gpu_server):
    """gamma=1, beta=0, mean=0, var=1-eps is the identity map."""
    rng = np.random.default_rng(1)
    C = 16
    x = _rand(rng, 3, 5, 5, C)
    eps = 1e-5
    ws = [np.ones(C, np.float32), np.zeros(C, np.float32), np.zeros(C, np.float32),
          np.full(C, 1.0 - eps, np.float32)]
    with OpSession(gpu_server, ws) as t:
        xv = t.act(x)
        yv = t.empty(x.nbytes)
        t.s.bn(t.fid, xv, yv, *t.w[:4], eps, 75, C)
        got = t.read(yv, x.shape)
    assert_close(got, x, 1e-6, "bn identity")


@pytest.mark.parametrize("n", [1, 4, 1023, 50000])
def test_elementwise(gpu_server, n):
    rng = np.random.default_rng(n)
    a, b = _rand(rng, n), _rand(rng, n)
    with OpSession(gpu_server, [np.zeros(4, np.float32)]) as t:
        av, bv = t.act(a), t.act(b)
        yv = t.empty(n * 4)
        t.s.launch(t.fid, OP_RELU, [av, yv], [n])
        np.testing.assert_array_equal(t.read(yv, (n,)), np.maximum(a, 0))
        t.s.launch(t.fid, OP_ADD, [av, bv, yv], [n, 0])
        np.testing.assert_array_equal(t.read(yv, (n,)), a + b)
        t.s.launch(t.fid, OP_ADD, [av, bv, yv], [n, 1])
        np.testing.assert_array_equal(t.read(yv, (n,)), np.maximum(a + b, 0))
        t.s.launch(t.fid, OP_GELU, [av, yv], [n])
        assert_close(t.read(yv, (n,)), ref.gelu(a), 2e-6, "gelu")
        t.s.launch(t.fid, OP_FILL, [yv], [n], [3.25])
        np.testing.assert_array_equal(t.read(yv, (n,)), np.full(n, 3.25, np.float32))
        t.s.launch(t.fid, OP_SUM, [av, yv], [n])
        assert_close(t.read(yv, (1,)), [a.astype(np.float64).sum()], 1e-4 if n > 1 else 1e-6, "sum")


def test_bias_act_and_layouts(gpu_server):
    rng = np.random.default_rng(3)
    x, bias = _rand(rng, 33, 50), _rand(rng, 50)
    img = _rand(rng, 2, 5, 37, 41)
    with OpSession(gpu_server, [bias]) as t:
        xv = t.act(x)
        yv = t.empty(x.nbytes)
        t.s.launch(t.fid, OP_BIAS_ACT, [xv, t.w[0], yv], [33, 50, ACT_RELU])
        np.testing.assert_array_equal(t.read(yv, x.shape), np.maximum(x + bias, 0))
        iv = t.act(img)
        ov = t.empty(img.nbytes)
        t.s.launch(t.fid, OP_NCHW_TO_NHWC, [iv, ov], [2, 5, 37, 41])
        nhwc = t.read(ov, (2, 37, 41, 5))
        np.testing.assert_array_equal(nhwc, img.transpose(0, 2, 3, 1))
        t.s.launch(t.fid, OP_NHWC_TO_NCHW, [ov, iv], [2, 5, 37, 41])
        np.testing.assert_array_equal(t.read(iv, img.shape), img)


@pytest.mark.parametrize("N,H,W,C", [(2, 40, 33, 70), (1, 112, 112, 96), (3, 16, 16, 8), (8, 7, 7, 2048), (2, 4, 4, 5),
                                     (2, 3, 5, 130)])
def test_global_avgpool_large_maps(gpu_server, N, H, W, C):
    """Maps of 16 pixels and more take the two-stage (sliced) reduction, smaller ones one thread
    per channel."""
    rng = np.random.default_rng(H + C)
    x = _rand(rng, N, H, W, C) + 0.5
    with OpSession(gpu_server, [np.zeros(4, np.float32)]) as t:
        xv = t.act(x)
        av = t.empty(N * C * 4)
        t.s.launch(t.fid, OP_AVGPOOL, [xv, av], [N, H * W, C, NHWC])
        got = t.read(av, (N, C))
        t.s.launch(t.fid, OP_AVGPOOL, [xv, av], [N, H * W, C, NHWC])
        again = t.read(av, (N, C))
    assert_close(got, ref.avgpool(x, nhwc=True), 2e-6, "global avgpool")
    np.testing.assert_array_equal(got, again)   # fixed summation order


def test_new_activations_window_average_and_strided_views(gpu_server):
    """relu6 / silu / sigmoid, k x k average pooling (also into a channel slice of a wider tensor),
    2-D strided copy, and batch-norm over the first channels of a wider tensor."""
    rng = np.random.default_rng(21)
    x, bias = _rand(rng, 17, 24) * 4, _rand(rng, 24)
    img = _rand(rng, 2, 9, 8, 12)
    g, b, mu = _rand(rng, 8), _rand(rng, 8), _rand(rng, 8)
    var = rng.uniform(0.2, 2.0, 8).astype(np.float32)
    with OpSession(gpu_server, [bias, g, b, mu, var]) as t:
        xv = t.act(x)
        yv = t.empty(x.nbytes)
        for act, name in ((ACT_RELU6, "relu6"), (ACT_SILU, "silu"), (ACT_SIGMOID, "sigmoid")):
            t.s.launch(t.fid, OP_BIAS_ACT, [xv, t.w[0], yv], [17, 24, act])
            assert_close(t.read(yv, x.shape), ref.activation(x + bias, name), 2e-6, name)
        iv = t.act(img)
        for k, st, pad in ((2, 2, 0), (3, 1, 1), (3, 2, 1)):
            want = ref.avgpool2d(img, k, st, pad)
            ov = t.empty(want.nbytes)
            t.s.launch(t.fid, OP_AVGPOOL2D, [iv, ov], [2, 9, 8, 12, k, st, pad, 0])
            assert_close(t.read(ov, want.shape), want, 2e-6, f"avgpool2d {k}/{st}/{pad}")
        # ... into channels 4..15 of a 20-channel tensor that holds a marker value elsewhere
        want = ref.avgpool2d(img, 2, 2, 0)
        wide = np.full(want.shape[:3] + (20,), 7.0, np.float32)
        wv = t.act(wide)
        t.s.launch(t.fid, OP_AVGPOOL2D, [iv, wv + 4 * 4], [2, 9, 8, 12, 2, 2, 0, 20])
        got = t.read(wv, wide.shape)
        assert_close(got[..., 4:16], want, 2e-6, "avgpool2d into a slice")
        assert (got[..., :4] == 7).all() and (got[..., 16:] == 7).all()
        # squeeze-and-excitation gating: every pixel of image n scaled per channel
        gate = rng.uniform(0, 1, (2, 12)).astype(np.float32)
        gv = t.act(gate)
        sv = t.empty(img.nbytes)
        t.s.launch(t.fid, OP_SCALE_CHANNELS, [iv, gv, sv], [2, 9 * 8, 12])
        np.testing.assert_array_equal(t.read(sv, img.shape), img * gate[:, None, None, :])
        # strided copy: columns 3..10 of x into columns 1..8 of a 12-wide matrix
        dst = np.zeros((17, 12), np.float32)
        dv = t.act(dst)
        t.s.launch(t.fid, OP_COPY2D, [xv + 3 * 4, dv + 1 * 4], [17, 8, 24, 12])
        got = t.read(dv, dst.shape)
        np.testing.assert_array_equal(got[:, 1:9], x[:, 3:11])
        assert (got[:, 0] == 0).all() and (got[:, 9:] == 0).all()
        # batch-norm + relu over the first 8 of 12 channels
        bv = t.empty(2 * 9 * 8 * 8 * 4)
        t.s.bn(t.fid, iv, bv, t.w[1], t.w[2], t.w[3], t.w[4], 1e-5, 2 * 9 * 8, 8, relu=True, x_pitch=12)
        want = ref.bn(np.ascontiguousarray(img[..., :8]), g, b, mu, var, 1e-5, 8, nhwc=True, relu=True)
        assert_close(t.read(bv, want.shape), want, 2e-6, "bn over a channel prefix")
        with pytest.raises(TorporError):   # pitch smaller than the channel count
            t.s.bn(t.fid, iv, bv, t.w[1], t.w[2], t.w[3], t.w[4], 1e-5, 2 * 9 * 8, 8, relu=True, x_pitch=4)
        with pytest.raises(TorporError):   # the view would run past the end of the source
            t.s.launch(t.fid, OP_COPY2D, [xv + 3 * 4, dv], [17, 8, 25, 12])
        with pytest.raises(TorporError):
            t.s.stream_synchronize(t.fid)


@pytest.mark.parametrize("C", [24, 10])          # NHWC: four channels per thread, and a count that path cannot take
@pytest.mark.parametrize("layout", [NHWC, NCHW])
def test_pooling(gpu_server, layout, C):
    rng = np.random.default_rng(9)
    N, H, W = 2, 15, 14
    x = _rand(rng, N, H, W, C) if layout == NHWC else _rand(rng, N, C, H, W)
    with OpSession(gpu_server, [np.zeros(4, np.float32)]) as t:
        xv = t.act(x)
        for k, stride, pad in ((3, 2, 1), (2, 2, 0), (3, 1, 1), (3, 2, 0)):
            want = ref.maxpool(x, k, stride, pad, nhwc=(layout == NHWC))
            yv = t.empty(want.nbytes)
            t.s.launch(t.fid, OP_MAXPOOL, [xv, yv], [N, H, W, C, k, stride, pad, layout])
            np.testing.assert_array_equal(t.read(yv, want.shape), want, err_msg=str((k, stride, pad)))
        av = t.empty(N * C * 4)
        t.s.launch(t.fid, OP_AVGPOOL, [xv, av], [N, H * W, C, layout])
        assert_close(t.read(av, (N, C)), ref.avgpool(x, nhwc=(layout == NHWC)), 2e-6, "avgpool")


@pytest.mark.parametrize("rows,width", [(128, 768), (5, 1024), (3, 50), (2, 4096), (1, 1), (7, 1540), (4, 2050), (3, 260), (2, 3000)])
def test_layernorm(gpu_server, rows, width):
    rng = np.random.default_rng(width)
    x, r = _rand(rng, rows, width) * 3 + 1, _rand(rng, rows, width)
    g, b = _rand(rng, width), _rand(rng, width)
    with OpSession(gpu_server, [g, b]) as t:
        xv, rv = t.act(x), t.act(r)
        yv = t.empty(x.nbytes)
        t.s.launch(t.fid, OP_LAYERNORM, [xv, rv, t.w[0], t.w[1], yv], [rows, width], [1e-12])
        got = t.read(yv, x.shape)
        t.s.launch(t.fid, OP_LAYERNORM, [xv, 0, t.w[0], t.w[1], yv], [rows, width], [1e-5])
        got2 = t.read(yv, x.shape)
    if width > 1:
        assert_close(got, ref.layernorm(x, r, g, b, 1e-12), 2e-5, "layernorm+res")
    assert_close(got2, ref.layernorm(x, None, g, b, 1e-5), 2e-5, "layernorm")


def test_layernorm_moments(gpu_server):
    """gamma=1, beta=0: every output row has mean 0 and variance 1."""
    rng = np.random.default_rng(0)
    x = _rand(rng, 16, 768) * 5 + 2
    with OpSession(gpu_server, [np.ones(768, np.float32), np.zeros(768, np.float32)]) as t:
        xv = t.act(x)
        yv = t.empty(x.nbytes)
        t.s.launch(t.fid, OP_LAYERNORM, [xv, 0, t.w[0], t.w[1], yv], [16, 768], [1e-12])
        y = t.read(yv, x.shape).astype(np.float64)
    assert np.abs(y.mean(1)).max() < 1e-5 and np.abs(y.var(1) - 1).max() < 1e-4


@pytest.mark.parametrize("rows,width,rpm", [(12 * 128, 128, 0), (2 * 4 * 96, 96, 4 * 96), (7, 384, 0), (3, 513, 0)])
def test_softmax(gpu_server, rows, width, rpm):
    rng = np.random.default_rng(width)
    x = _rand(rng, rows, width) * 4
    mask = None
    if rpm:
        mask = np.where(rng.random((rows // rpm, width)) < 0.2, np.float32(-1e30), np.float32(0)).astype(np.float32)
        mask[:, 0] = 0
    with OpSession(gpu_server, [np.zeros(4, np.float32)]) as t:
        xv = t.act(x)
        mv = t.act(mask) if mask is not None else 0
        yv = t.empty(x.nbytes)
        t.s.launch(t.fid, OP_SOFTMAX, [xv, mv, yv], [rows, width, rpm], [0.125])
        got = t.read(yv, x.shape)
    want = ref.softmax(x, mask, 0.125, rpm if rpm else 1)
    assert_close(got, want, 2e-6, "softmax")
    assert np.abs(got.astype(np.float64).sum(1) - 1).max() < 1e-5
    if mask is not None:
        assert (got[np.repeat(mask, rpm, axis=0) < -1] == 0).all()


@pytest.mark.parametrize("B,A,S,packed,masked", [
    (1, 12, 128, True, False),    # BERT-base shape, heads read from a [tokens, 3H] projection
    (2, 16, 384, True, False),    # BERT-large shape (batch 2), 96 heads-times-blocks per XCD
    (2, 3, 100, False, True),     # ragged sequence (padded keys and queries), key mask, no XCD remap
    (1, 8, 32, False, True),      # a single key block: three of the four wavefronts idle
    (3, 1, 7, False, False),      # shorter than one block
])
def test_attention(gpu_server, B, A, S, packed, masked):
    rng = np.random.default_rng(S + A)
    dh, H = 64, A * 64
    scale = 0.125
    if packed:
        qkv = _rand(rng, B * S, 3 * H)
        q, k, v = (qkv[:, i * H:(i + 1) * H].reshape(B, S, A, dh) for i in range(3))
    else:
        q, k, v = (_rand(rng, B, S, A, dh) * 2 for _ in range(3))
    mask = None
    if masked:
        mask = np.where(rng.random((B, S)) < 0.25, np.float32(-1e4), np.float32(0)).astype(np.float32)
        mask[:, 0] = 0
    with OpSession(gpu_server, [np.zeros(4, np.float32)]) as t:
        if packed:
            base = t.act(qkv)
            ptrs, ld = [base, base + H * 4, base + 2 * H * 4], 3 * H
        else:
            ptrs, ld = [t.act(np.ascontiguousarray(x)) for x in (q, k, v)], H
        mv = t.act(mask) if mask is not None else 0
        ov = t.empty(B * S * H * 4)
        t.s.launch(t.fid, OP_ATTENTION, ptrs + [mv, ov], [B, A, S, dh, ld, ld, ld, H], [scale])
        assert t.s.last_kernel() == "attention_32q_dh64"
        got = t.read(ov, (B, S, A, dh))
        # unsupported head width and out-of-span operands are refused, not launched
        with pytest.raises(TorporError):
            t.s.launch(t.fid, OP_ATTENTION, ptrs + [mv, ov], [B, A * 2, S, 32, ld, ld, ld, H], [scale])
        with pytest.raises(TorporError):
            t.s.launch(t.fid, OP_ATTENTION, ptrs + [mv, ov], [B, A, S + 1, dh, ld, ld, ld, H], [scale])
        with pytest.raises(TorporError):
            t.s.stream_synchronize(t.fid)   # refused ops are reported once more at the next sync
    assert_close(got, ref.attention(q, k, v, mask, scale), 2e-5, "attention")


@pytest.mark.parametrize("H", [96, 1024, 37])     # one float4 pass, several, and a width the float4 path cannot take
def test_embedding(gpu_server, H):
    rng = np.random.default_rng(2)
    V, P, T, B, S = 100, 40, 2, 3, 17
    word, pos, typ = _rand(rng, V, H), _rand(rng, P, H), _rand(rng, T, H)
    ids = rng.integers(0, V, (B, S)).astype(np.int64)
    tids = rng.integers(0, T, (B, S)).astype(np.int64)
    with OpSession(gpu_server, [word, pos, typ]) as t:
        iv, tv = t.act(ids), t.act(tids)
        yv = t.empty(B * S * H * 4)
        t.s.launch(t.fid, OP_EMBEDDING, [iv, tv, t.w[0], t.w[1], t.w[2], yv], [B * S, S, H, V, T])
        got = t.read(yv, (B * S, H))
        t.s.launch(t.fid, OP_EMBEDDING, [iv, 0, t.w[0], t.w[1], t.w[2], yv], [B * S, S, H, V, T])
        got0 = t.read(yv, (B * S, H))
    assert_close(got, ref.embedding(ids, tids, word, pos, typ, S), 1e-6, "embedding")
    assert_close(got0, ref.embedding(ids, None, word, pos, typ, S), 1e-6, "embedding type 0")
    # the vector and the scalar path add in the same order, (word + position) + type in float32
    p_rows = pos[np.arange(B * S) % S]
    assert np.array_equal(got, (word[ids.ravel()] + p_rows) + typ[tids.ravel()])
    assert np.array_equal(got0, (word[ids.ravel()] + p_rows) + typ[0])
