"""Convolution kernels vs the direct-loop fp64 C oracle, through the C-ABI (reference call site
cudnnConvolutionForward, include/server/cuda_server.hpp:708-735)."""
import numpy as np
import pytest

from oracle import ops as ref
from tests.harness import OpSession, assert_close
from torpor_amd.server import ACT_NONE, ACT_RELU, NCHW, NHWC, TorporError

pytestmark = pytest.mark.gpu
RTOL = 3e-5


def _rand(rng, *shape):
    return rng.standard_normal(shape).astype(np.float32)


CASES = [
    # N, H, W, Cin, Cout, k, stride, pad, x_layout, y_layout, expected kernel
    (1, 56, 56, 64, 64, 1, 1, 0, NHWC, NHWC, "gemm_fast"),        # 1x1
    (2, 28, 28, 256, 512, 1, 2, 0, NHWC, NHWC, "gemm_fast"),      # 1x1 stride 2 (downsample)
    (1, 56, 56, 64, 64, 3, 1, 1, NHWC, NHWC, "conv3x3_wino"),     # 3x3 stride 1: Winograd
    (1, 28, 28, 128, 128, 3, 1, 1, NHWC, NHWC, "conv3x3_fast"),   # the same kind of layer at batch 1: below the Winograd path's size bound
    (1, 20, 20, 24, 40, 3, 1, 1, NHWC, NHWC, "conv3x3_fast"),     # 3x3 stride 1 whose channel counts the Winograd path does not take
    (2, 28, 28, 128, 128, 3, 2, 1, NHWC, NHWC, "conv3x3_fast"),   # 3x3 stride 2
    (1, 7, 7, 512, 512, 3, 1, 1, NHWC, NHWC, "conv3x3_wino"),     # tiny odd map (edge tiles), split over channels
    (8, 28, 28, 128, 128, 3, 1, 1, NHWC, NHWC, "conv3x3_wino"),   # batch 8
    (8, 14, 14, 256, 256, 3, 1, 1, NHWC, NHWC, "conv3x3_wino"),   # the dominant ResNet-152 batch 8 layer: 392 tiles, ragged last block
    (3, 15, 13, 16, 32, 3, 1, 1, NHWC, NHWC, "conv3x3_wino"),     # odd height and width, one K-block, one channel block
    (2, 9, 10, 48, 96, 3, 1, 1, NHWC, NHWC, "conv3x3_wino"),      # three K-blocks, three channel blocks
    (1, 64, 64, 3, 64, 7, 2, 3, NCHW, NHWC, "conv_stem7x7"),      # stem: NCHW in, NHWC out
    (1, 64, 64, 3, 48, 7, 2, 3, NCHW, NHWC, "conv_generic"),      # a stem whose channel count the stem kernel does not take
    (1, 13, 11, 5, 7, 3, 1, 1, NCHW, NCHW, "conv_generic"),       # odd sizes, NCHW both
    (1, 9, 9, 12, 20, 5, 2, 2, NHWC, NCHW, "conv_generic"),       # 5x5, mixed layouts
    (1, 10, 10, 12, 16, 3, 1, 0, NHWC, NHWC, "conv_generic"),     # Cin % 8 != 0
    (2, 12, 12, 48, 64, 5, 1, 2, NHWC, NHWC, "conv_generic"),     # Inception's 5x5
]


@pytest.mark.parametrize("N,H,W,Cin,Cout,k,stride,pad,xl,yl,kern", CASES)
def test_conv(gpu_server, monkeypatch, N, H, W, Cin, Cout, k, stride, pad, xl, yl, kern):
    if kern.startswith("conv3x3_wino"):
        monkeypatch.setenv("TORPOR_WINO_MIN_GFLOP", "0")      # the Winograd path also for layers below its size bound
    rng = np.random.default_rng(N + H * 3 + Cin * 5 + Cout * 7 + k)
    x_nchw = _rand(rng, N, Cin, H, W)
    w = _rand(rng, Cout, Cin, k, k) * np.float32(1.0 / np.sqrt(Cin * k * k))
    x = x_nchw if xl == NCHW else np.ascontiguousarray(x_nchw.transpose(0, 2, 3, 1))
    Ho, Wo = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    with OpSession(gpu_server, [w]) as t:
        xv = t.act(x)
        yv = t.empty(N * Ho * Wo * Cout * 4)
        t.s.conv(t.fid, xv, t.w[0], yv, N, H, W, Cin, Cout, k, k, stride=stride, pad=pad, x_layout=xl, y_layout=yl)
        assert t.s.last_kernel().startswith(kern), t.s.last_kernel()
        got = t.read(yv, (N, Ho, Wo, Cout) if yl == NHWC else (N, Cout, Ho, Wo))
    want = ref.conv2d(x, w, (stride, stride), (pad, pad), x_nhwc=(xl == NHWC), y_nhwc=(yl == NHWC))
    assert_close(got, want, RTOL, f"conv {k}x{k} s{stride}")


@pytest.mark.parametrize("splits", [1, 2, 3, 8])
def test_winograd_split_over_channels_and_direct_kernel_agree(gpu_server, monkeypatch, splits):
    """Winograd F(2x2, 3x3) with its input channels split 1 / 2 / 3 / 8 ways (summed inside the launch, in slot
    order) against the oracle and against the direct kernel on the same operands; pitched input and output
    (a channel slice of wider tensors, as the DenseNets use them) and the fused batch-norm + residual + ReLU."""
    rng = np.random.default_rng(40 + splits)
    N, H, W, Cin, Cout, XP, YP = 2, 14, 14, 128, 64, 160, 96
    xw = _rand(rng, N, H, W, XP)
    w = _rand(rng, Cout, Cin, 3, 3) * np.float32(1.0 / np.sqrt(Cin * 9))
    g, b, mu = _rand(rng, Cout), _rand(rng, Cout), _rand(rng, Cout)
    var = rng.uniform(0.5, 2.0, Cout).astype(np.float32)
    res = _rand(rng, N, H, W, Cout)                        # the residual is a dense tensor of its own
    x = np.ascontiguousarray(xw[..., :Cin])
    outs = {}
    for path in ("wino", "direct"):
        monkeypatch.setenv("TORPOR_WINOGRAD", "1" if path == "wino" else "0")
        monkeypatch.setenv("TORPOR_WINO_SPLITS", str(splits))
        monkeypatch.setenv("TORPOR_WINO_MIN_GFLOP", "0")
        with OpSession(gpu_server, [w, g, b, mu, var]) as t:
            xv, rv = t.act(xw), t.act(res)
            yv = t.act(np.full((N, H, W, YP), 7.0, np.float32))
            t.s.conv(t.fid, xv, t.w[0], yv, N, H, W, Cin, Cout, 3, 3, stride=1, pad=1, x_pitch=XP, y_pitch=YP,
                     bn=tuple(t.w[1:5]), bn_eps=1e-5, residual=rv, act=ACT_RELU)
            assert t.s.last_kernel().startswith("conv3x3_wino" if path == "wino" else "conv3x3_fast"), t.s.last_kernel()
            outs[path] = t.read(yv, (N, H, W, YP))
    z = ref.conv2d(x, w, (1, 1), (1, 1), x_nhwc=True, y_nhwc=True)
    z = ref.bn(z, g, b, mu, var, 1e-5, Cout, nhwc=True).astype(np.float64) + res
    for path, got in outs.items():
        assert_close(got[..., :Cout], np.maximum(z, 0), 5e-5, f"{path} conv+bn+res+relu, pitched")
        assert np.all(got[..., Cout:] == 7.0), f"{path}: wrote outside its channel slice"
    assert_close(outs["wino"][..., :Cout], outs["direct"][..., :Cout], 5e-5, "Winograd against the direct kernel")


def test_winograd_is_deterministic_and_keeps_non_finite_values_local(gpu_server, monkeypatch):
    """Two runs give the same bits (the split is summed in slot order), and an infinity in the input reaches
    exactly the outputs whose 3x3 window holds it."""
    monkeypatch.setenv("TORPOR_WINO_MIN_GFLOP", "0")
    rng = np.random.default_rng(9)
    N, H, W, C = 1, 12, 12, 32
    x = _rand(rng, N, H, W, C)
    x[0, 5, 6, :] = np.inf
    w = np.abs(_rand(rng, C, C, 3, 3)) + np.float32(0.1)       # positive filters: the window's sum is +inf, never inf - inf
    with OpSession(gpu_server, [w]) as t:
        xv = t.act(x)
        yv = t.empty(x.nbytes)
        runs = []
        for _ in range(2):
            t.s.conv(t.fid, xv, t.w[0], yv, N, H, W, C, C, 3, 3, stride=1, pad=1)
            assert t.s.last_kernel().startswith("conv3x3_wino")
            runs.append(t.read(yv, (N, H, W, C)))
    assert np.array_equal(runs[0], runs[1], equal_nan=True)
    touched = np.zeros((H, W), bool)
    touched[4:7, 5:8] = True
    assert np.all(np.isfinite(runs[0][0][~touched])), "an infinity left the windows that hold it"
    assert not np.any(np.isfinite(runs[0][0][touched]))
    xf = x.copy()
    xf[0, 5, 6, :] = 0.0
    z = ref.conv2d(xf, w, (1, 1), (1, 1), x_nhwc=True, y_nhwc=True)
    assert_close(runs[0][0][~touched], z[0][~touched], RTOL, "outputs away from the infinite pixel")


@pytest.mark.parametrize("k,Cin,Cout,HW", [(1, 64, 256, 14), (3, 64, 64, 14), (7, 3, 16, 20)])
def test_conv_bn_residual_relu(gpu_server, k, Cin, Cout, HW):
    """The fused epilogue of a bottleneck's last convolution: relu(bn(conv(x)) + identity)."""
    rng = np.random.default_rng(k)
    N, pad = 2, k // 2
    x = _rand(rng, N, HW, HW, Cin)
    w = _rand(rng, Cout, Cin, k, k) * np.float32(1.0 / np.sqrt(Cin * k * k))
    g, b, mu = _rand(rng, Cout), _rand(rng, Cout), _rand(rng, Cout)
    var = rng.uniform(0.5, 2.0, Cout).astype(np.float32)
    res = _rand(rng, N, HW, HW, Cout)
    with OpSession(gpu_server, [w, g, b, mu, var]) as t:
        xv, rv = t.act(x), t.act(res)
        yv = t.empty(res.nbytes)
        t.s.conv(t.fid, xv, t.w[0], yv, N, HW, HW, Cin, Cout, k, k, stride=1, pad=pad, bn=tuple(t.w[1:5]),
                 bn_eps=1e-5, residual=rv, act=ACT_RELU)
        got = t.read(yv, res.shape)
    z = ref.conv2d(x, w, (1, 1), (pad, pad), x_nhwc=True, y_nhwc=True)
    z = ref.bn(z, g, b, mu, var, 1e-5, Cout, nhwc=True).astype(np.float64) + res
    assert_close(got, np.maximum(z, 0), 5e-5, "conv+bn+res+relu")


@pytest.mark.parametrize("N,H,W,Cout,xl,yl", [
    (1, 224, 224, 64, NCHW, NHWC),      # the served shape
    (2, 30, 29, 64, NCHW, NHWC),        # odd output height (15): the second row of the last pair does not exist
    (1, 70, 75, 128, NCHW, NHWC),       # two channel blocks; 38 output columns: a full block and a ragged one
    (2, 33, 64, 64, NHWC, NHWC),        # channels-last input
    (1, 40, 36, 64, NCHW, NCHW),        # NCHW output (the element-wise write-out)
])
def test_stem_convolution(gpu_server, N, H, W, Cout, xl, yl):
    """7x7 stride 2 padding 3 from 3 channels (cudnnConvolutionForward of the ResNet / DenseNet stem,
    cuda_server.hpp:708-735) with the batch-norm + ReLU that follows it fused, against the direct-loop oracle."""
    rng = np.random.default_rng(H * 7 + W + Cout)
    x_nchw = _rand(rng, N, 3, H, W)
    w = _rand(rng, Cout, 3, 7, 7) * np.float32(1.0 / np.sqrt(147))
    g, b, mu = _rand(rng, Cout), _rand(rng, Cout), _rand(rng, Cout)
    var = rng.uniform(0.5, 2.0, Cout).astype(np.float32)
    x = x_nchw if xl == NCHW else np.ascontiguousarray(x_nchw.transpose(0, 2, 3, 1))
    Ho, Wo = (H + 6 - 7) // 2 + 1, (W + 6 - 7) // 2 + 1
    shape = (N, Ho, Wo, Cout) if yl == NHWC else (N, Cout, Ho, Wo)
    with OpSession(gpu_server, [w, g, b, mu, var]) as t:
        xv = t.act(x)
        guard = np.full(shape, 7.0, np.float32)
        yv = t.act(np.concatenate([guard.ravel(), np.full(64, 7.0, np.float32)]))   # 64 floats behind y must stay
        t.s.conv(t.fid, xv, t.w[0], yv, N, H, W, 3, Cout, 7, 7, stride=2, pad=3, x_layout=xl, y_layout=yl)
        assert t.s.last_kernel().startswith("conv_stem7x7"), t.s.last_kernel()
        plain = t.read(yv, shape)
        tail = t.read(yv + guard.nbytes, (64,))
        t.s.conv(t.fid, xv, t.w[0], yv, N, H, W, 3, Cout, 7, 7, stride=2, pad=3, x_layout=xl, y_layout=yl,
                 bn=tuple(t.w[1:5]), bn_eps=1e-5, act=ACT_RELU)
        fused = t.read(yv, shape)
    z = ref.conv2d(x, w, (2, 2), (3, 3), x_nhwc=(xl == NHWC), y_nhwc=(yl == NHWC))
    assert_close(plain, z, RTOL, "stem")
    assert np.all(tail == 7.0), "stem wrote past the end of its output"
    zb = ref.bn(z, g, b, mu, var, 1e-5, Cout, hw=Ho * Wo, nhwc=(yl == NHWC))
    assert_close(fused, np.maximum(zb, 0), 5e-5, "stem+bn+relu")


def test_stem_keeps_an_infinity_out_of_rows_whose_receptive_field_does_not_hold_it(gpu_server):
    """The stem kernel pads its 7 filter rows to 8 MFMA steps per lane half; the step that has no filter row must
    contribute nothing, also when the input row it would meet holds Inf (0 * Inf is NaN).  Input row 24 is
    infinite: output rows 11..13 see it (2*ho-3 <= 24 <= 2*ho+3), every other row must equal the oracle's."""
    rng = np.random.default_rng(5)
    x = _rand(rng, 1, 3, 64, 64)
    x[:, :, 24, :] = np.inf
    w = _rand(rng, 64, 3, 7, 7) * np.float32(1.0 / np.sqrt(147))
    with OpSession(gpu_server, [w]) as t:
        xv = t.act(x)
        yv = t.empty(32 * 32 * 64 * 4)
        t.s.conv(t.fid, xv, t.w[0], yv, 1, 64, 64, 3, 64, 7, 7, stride=2, pad=3, x_layout=NCHW, y_layout=NHWC)
        assert t.s.last_kernel().startswith("conv_stem7x7"), t.s.last_kernel()
        got = t.read(yv, (1, 32, 32, 64))
    x_fin = x.copy()
    x_fin[:, :, 24, :] = 0.0
    z = ref.conv2d(x_fin, w, (2, 2), (3, 3), x_nhwc=False, y_nhwc=True)
    clean = [ho for ho in range(32) if not (2 * ho - 3 <= 24 <= 2 * ho + 3)]
    assert clean == [r for r in range(32) if r not in (11, 12, 13)]
    assert np.all(np.isfinite(got[:, clean])), "an infinity outside the receptive field reached the output"
    assert_close(got[:, clean], z[:, clean], RTOL, "stem rows away from the infinite input row")
    assert not np.any(np.isfinite(got[:, 11:14])), "rows that do read the infinite row"


def test_conv_identities(gpu_server):
    """Closed forms: a centred delta kernel is the identity; an all-ones 3x3 kernel on an all-ones
    image counts the in-bounds taps (4 / 6 / 9 at corner / edge / interior)."""
    C, HW = 8, 12
    rng = np.random.default_rng(0)
    x = _rand(rng, 1, HW, HW, C)
    delta = np.zeros((C, C, 3, 3), np.float32)
    for c in range(C):
        delta[c, c, 1, 1] = 1.0
    ones_w = np.ones((C, C, 3, 3), np.float32)
    with OpSession(gpu_server, [delta, ones_w]) as t:
        xv, ov = t.act(x), t.act(np.ones_like(x))
        yv = t.empty(x.nbytes)
        t.s.conv(t.fid, xv, t.w[0], yv, 1, HW, HW, C, C, 3, 3, stride=1, pad=1)
        got = t.read(yv, x.shape)
        np.testing.assert_array_equal(got, x)
        t.s.conv(t.fid, ov, t.w[1], yv, 1, HW, HW, C, C, 3, 3, stride=1, pad=1)
        cnt = t.read(yv, x.shape)
    assert cnt[0, 0, 0, 0] == 4 * C and cnt[0, 0, 5, 0] == 6 * C and cnt[0, 5, 5, 0] == 9 * C


def test_conv_rejects_bad_shapes(gpu_server):
    from torpor_amd._lib import TorporError
    w = np.zeros((8, 8, 3, 3), np.float32)
    with OpSession(gpu_server, [w]) as t:
        xv = t.act(np.zeros((1, 6, 6, 8), np.float32))
        yv = t.empty(1 * 6 * 6 * 8 * 4)
        with pytest.raises(TorporError):   # claims a larger input than the buffer holds
            t.s.conv(t.fid, xv, t.w[0], yv, 1, 8, 8, 8, 8, 3, 3, stride=1, pad=1)
        with pytest.raises(TorporError):   # claims more filters than uploaded
            t.s.conv(t.fid, xv, t.w[0], yv, 1, 6, 6, 8, 16, 3, 3, stride=1, pad=1)
        with pytest.raises(TorporError):   # a group count that does not divide the channels
            t.s.conv(t.fid, xv, t.w[0], yv, 1, 6, 6, 8, 8, 3, 3, stride=1, pad=1, groups=3)
        with pytest.raises(TorporError):
            t.s.stream_synchronize(t.fid)
        t.s.conv(t.fid, xv, t.w[0], yv, 1, 6, 6, 8, 8, 3, 3, stride=1, pad=1)


@pytest.mark.parametrize("kh,kw,stride,Cin,Cout,H,W", [
    (1, 7, 1, 16, 24, 17, 17), (7, 1, 1, 48, 70, 17, 17), (1, 3, 1, 24, 40, 8, 8), (3, 1, 1, 16, 64, 8, 9),
    (1, 7, 1, 256, 32, 5, 7),   # splits over channels
    (1, 7, 1, 40, 48, 17, 17), (7, 1, 1, 40, 48, 17, 17),   # 32x32 tiles, one wavefront per tap, 8 channels per K-block
    (1, 3, 1, 40, 40, 8, 8), (3, 1, 1, 64, 64, 8, 9),       # ... three taps: 8 and 16 channels per K-block
    (1, 7, 1, 64, 256, 64, 64),                              # a grid that fills the chip stays on 64x64 tiles
])
def test_conv_tap_shapes(gpu_server, kh, kw, stride, Cin, Cout, H, W):
    """The asymmetric convolutions of Inception on the MFMA taps kernel ("same" padding),
    with the fused batch-norm + ReLU of a BasicConv2d."""
    rng = np.random.default_rng(kh * 10 + kw + Cin)
    N, ph, pw = 2, kh // 2, kw // 2
    x = _rand(rng, N, H, W, Cin)
    w = _rand(rng, Cout, Cin, kh, kw) * np.float32(1.0 / np.sqrt(Cin * kh * kw))
    g, b, mu = _rand(rng, Cout), _rand(rng, Cout), _rand(rng, Cout)
    var = rng.uniform(0.5, 2.0, Cout).astype(np.float32)
    Ho, Wo = (H + 2 * ph - kh) // stride + 1, (W + 2 * pw - kw) // stride + 1
    with OpSession(gpu_server, [w, g, b, mu, var]) as t:
        xv = t.act(x)
        yv = t.empty(N * Ho * Wo * Cout * 4)
        t.s.conv(t.fid, xv, t.w[0], yv, N, H, W, Cin, Cout, kh, kw, stride=stride, pad=(ph, pw))
        # few tiles and at least 32 input channels: 32x32 tiles with one wavefront per tap; else 64x64 tiles
        small = Cin >= 32 and -(-N * Ho * Wo // 64) * -(-Cout // 64) < 128
        want = f"conv_taps_{kh}x{kw}_32x32_k{kh * kw}" if small else f"conv_taps_{kh}x{kw}_64x64"
        assert t.s.last_kernel() == want, (t.s.last_kernel(), want)
        plain = t.read(yv, (N, Ho, Wo, Cout))
        t.s.conv(t.fid, xv, t.w[0], yv, N, H, W, Cin, Cout, kh, kw, stride=stride, pad=(ph, pw), bn=tuple(t.w[1:5]),
                 bn_eps=1e-3, act=ACT_RELU)
        fused = t.read(yv, (N, Ho, Wo, Cout))
    want = ref.conv2d(x, w, (stride, stride), (ph, pw), x_nhwc=True, y_nhwc=True)
    assert_close(plain, want, RTOL, f"conv {kh}x{kw}")
    z = ref.bn(want, g, b, mu, var, 1e-3, Cout, nhwc=True, relu=True)
    assert_close(fused, z, 5e-5, f"conv {kh}x{kw} + bn + relu")


@pytest.mark.parametrize("C,k,stride,HW", [(32, 3, 1, 14), (24, 3, 2, 15), (16, 5, 2, 9), (8, 3, 1, 5), (12, 7, 1, 9),
                                           (40, 5, 1, 6)])
def test_depthwise(gpu_server, C, k, stride, HW):
    """groups == channels (MobileNet-style), with the fused batch-norm + relu6 epilogue."""
    from torpor_amd.server import ACT_RELU6
    rng = np.random.default_rng(C + k)
    N, pad = 2, k // 2
    x = _rand(rng, N, HW, HW, C) * 2
    w = _rand(rng, C, 1, k, k)
    g, b, mu = _rand(rng, C), _rand(rng, C), _rand(rng, C)
    var = rng.uniform(0.5, 2.0, C).astype(np.float32)
    Ho = (HW + 2 * pad - k) // stride + 1
    with OpSession(gpu_server, [w, g, b, mu, var]) as t:
        xv = t.act(x)
        yv = t.empty(N * Ho * Ho * C * 4)
        t.s.conv(t.fid, xv, t.w[0], yv, N, HW, HW, C, C, k, k, stride=stride, pad=pad, groups=C)
        # 3x3 / 5x5 run the branch-free vector kernel, other sizes the general one
        assert t.s.last_kernel() == {3: "depthwise_3x3", 5: "depthwise_5x5"}.get(k, "depthwise_nhwc")
        plain = t.read(yv, (N, Ho, Ho, C))
        t.s.conv(t.fid, xv, t.w[0], yv, N, HW, HW, C, C, k, k, stride=stride, pad=pad, groups=C,
                 bn=tuple(t.w[1:5]), bn_eps=1e-5, act=ACT_RELU6)
        fused = t.read(yv, (N, Ho, Ho, C))
        with pytest.raises(TorporError):   # a group count that does not divide the channels
            t.s.conv(t.fid, xv, t.w[0], yv, N, HW, HW, C, C, k, k, stride=stride, pad=pad, groups=7)
        with pytest.raises(TorporError):
            t.s.stream_synchronize(t.fid)
    want = ref.depthwise_conv2d(x, w, (stride, stride), (pad, pad))
    assert_close(plain, want, RTOL, "depthwise")
    z = ref.bn(want, g, b, mu, var, 1e-5, C, nhwc=True)
    assert_close(fused, ref.activation(z, "relu6"), 5e-5, "depthwise+bn+relu6")


@pytest.mark.parametrize("Cin,Cout,groups,k,stride,HW", [(64, 128, 4, 3, 1, 14), (32, 32, 2, 1, 1, 9), (24, 36, 3, 3, 2, 11),
                                                         (6, 10, 2, 5, 1, 8), (128, 128, 32, 3, 1, 7)])
def test_grouped_convolution(gpu_server, Cin, Cout, groups, k, stride, HW):
    """cudnnSetConvolutionGroupCount (cuda_server.hpp:671) with groups that are not the channel count (ResNeXt-style):
    against torch's float64 grouped convolution, and against the fp64 oracle applied group by group; with the
    fused bias + residual + relu epilogue on top."""
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(Cin + Cout + groups)
    N, pad = 2, k // 2
    x = _rand(rng, N, HW, HW, Cin)
    w = _rand(rng, Cout, Cin // groups, k, k)
    bias = _rand(rng, Cout)
    Ho = (HW + 2 * pad - k) // stride + 1
    res = _rand(rng, N, Ho, Ho, Cout)
    with OpSession(gpu_server, [w, bias]) as t:
        xv = t.act(x)
        rv = t.act(res)
        yv = t.empty(N * Ho * Ho * Cout * 4)
        t.s.conv(t.fid, xv, t.w[0], yv, N, HW, HW, Cin, Cout, k, k, stride=stride, pad=pad, groups=groups)
        plain = t.read(yv, (N, Ho, Ho, Cout))
        t.s.conv(t.fid, xv, t.w[0], yv, N, HW, HW, Cin, Cout, k, k, stride=stride, pad=pad, groups=groups,
                 bias=t.w[1], residual=rv, act=ACT_RELU)
        fused = t.read(yv, (N, Ho, Ho, Cout))
        with pytest.raises(TorporError):   # grouped and not depthwise needs NHWC on both sides
            t.s.conv(t.fid, xv, t.w[0], yv, N, HW, HW, Cin, Cout, k, k, stride=stride, pad=pad, groups=groups,
                     x_layout=NCHW)
        with pytest.raises(TorporError):
            t.s.stream_synchronize(t.fid)
    want64 = F.conv2d(torch.from_numpy(x).double().permute(0, 3, 1, 2), torch.from_numpy(w).double(), stride=stride,
                      padding=pad, groups=groups).permute(0, 2, 3, 1).numpy()
    assert_close(plain, want64.astype(np.float32), RTOL, "grouped conv vs torch float64")
    cig, cog = Cin // groups, Cout // groups
    per_group = [ref.conv2d(np.ascontiguousarray(x[..., g * cig:(g + 1) * cig]), np.ascontiguousarray(w[g * cog:(g + 1) * cog]),
                            (stride, stride), (pad, pad), x_nhwc=True, y_nhwc=True) for g in range(groups)]
    want = np.concatenate(per_group, axis=-1)
    assert_close(plain, want, RTOL, "grouped conv vs the oracle, group by group")
    assert_close(fused, np.maximum(want + bias + res, 0).astype(np.float32), 5e-5, "grouped conv + bias + residual + relu")


@pytest.mark.parametrize("k", [1, 3])
def test_conv_channel_slices(gpu_server, k):
    """DenseNet-style concatenation without copies: read the first Cin channels of a wider
    tensor (x_pitch) and write Cout channels into a slice of another (y_pitch, pointer offset)."""
    rng = np.random.default_rng(k)
    N, HW, Cin, Cout, XP, YP, off = 2, 12, 32, 16, 48, 40, 8
    xw = _rand(rng, N, HW, HW, XP)
    w = _rand(rng, Cout, Cin, k, k) * np.float32(1.0 / np.sqrt(Cin * k * k))
    ywide = np.full((N, HW, HW, YP), 3.0, np.float32)
    with OpSession(gpu_server, [w]) as t:
        xv, yv = t.act(xw), t.act(ywide)
        t.s.conv(t.fid, xv, t.w[0], yv + off * 4, N, HW, HW, Cin, Cout, k, k, stride=1, pad=k // 2, x_pitch=XP,
                 y_pitch=YP)
        got = t.read(yv, ywide.shape)
        with pytest.raises(TorporError):   # slice would run past the end of y
            t.s.conv(t.fid, xv, t.w[0], yv + (YP - Cout + 1) * 4, N, HW, HW, Cin, Cout, k, k, stride=1, pad=k // 2,
                     x_pitch=XP, y_pitch=YP)
        with pytest.raises(TorporError):
            t.s.stream_synchronize(t.fid)
    want = ref.conv2d(np.ascontiguousarray(xw[..., :Cin]), w, (1, 1), (k // 2, k // 2), x_nhwc=True, y_nhwc=True)
    assert_close(got[..., off:off + Cout], want, RTOL, "conv into a channel slice")
    assert (got[..., :off] == 3).all() and (got[..., off + Cout:] == 3).all()


@pytest.mark.parametrize("cfg,name", [(0, "fast_128x128"), (1, "fast_64x64"), (2, "fast_64x64_k3"), (3, "fast_32x32_k9"),
                                      (4, "fast_32x32_k3")])
def test_forced_conv3x3_configs(cfg, name):
    """Every tile shape of the 3x3 kernel, including those whose wavefronts split the K-block
    (TORPOR_CONV3_CFG forces one; read once per process, hence the subprocess): ragged pixel
    counts, ragged output channels, stride 2, one and several channel blocks."""
    import os
    import subprocess
    import sys
    code = r'''
import numpy as np, sys
from oracle import ops as ref
from torpor_amd.server import Server
from tests.harness import OpSession, assert_close
rng = np.random.default_rng(1)
with Server(mem_limit_bytes=1 << 30, pool_bytes=2 << 30) as s:
    for (N, H, W, Cin, Cout, stride) in [(1, 14, 14, 64, 64, 1), (2, 9, 7, 8, 40, 1), (1, 15, 15, 48, 72, 2), (3, 7, 7, 256, 96, 1),
                                         (2, 16, 16, 64, 32, 2), (1, 56, 56, 32, 64, 1), (5, 5, 3, 96, 70, 1)]:
        x = rng.standard_normal((N, H, W, Cin)).astype(np.float32)
        w = (rng.standard_normal((Cout, Cin, 3, 3)) / np.sqrt(Cin * 9)).astype(np.float32)
        Ho, Wo = (H + 2 - 3) // stride + 1, (W + 2 - 3) // stride + 1
        with OpSession(s, [w]) as t:
            xv = t.act(x)
            yv = t.empty(N * Ho * Wo * Cout * 4)
            s.conv(t.fid, xv, t.w[0], yv, N, H, W, Cin, Cout, 3, 3, stride=stride, pad=1)
            assert s.last_kernel() == "conv3x3_" + sys.argv[1], s.last_kernel()
            got = t.read(yv, (N, Ho, Wo, Cout))
        want = ref.conv2d(x, w, (stride, stride), (1, 1), x_nhwc=True, y_nhwc=True)
        assert_close(got, want, 3e-5, "conv3x3 " + sys.argv[1])
print("ok")
'''
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, TORPOR_CONV3_CFG=str(cfg), TORPOR_WINOGRAD="0", PYTHONPATH=root)   # the direct kernels are meant
    r = subprocess.run([sys.executable, "-c", code, name], env=env, cwd=root, capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0 and "ok" in r.stdout, r.stdout + r.stderr


# ---------------------------------------------------------------- batch-norm + ReLU on the input of a 1x1 convolution
@pytest.mark.parametrize("rows,cin,cout,ctot,post", [
    (196, 256, 128, 640, True),     # DenseNet block 3: K a multiple of 128 -> 32x32 tiles
    (196, 224, 128, 640, True),     # K not a multiple of 64: 64x64 tiles, K-blocks of 32
    (196, 288, 128, 640, True),     # 32x32 tiles with half a K-block at the end (4.5 blocks of 64)
    (49, 1888, 128, 1920, True),    # ... 29.5 blocks, split over workgroups: the last slice ends with the half block
    (196, 416, 128, 640, True),     # ... 6.5 blocks
    (3136, 64, 128, 256, True),     # first layer of block 1: two K-blocks, many rows
    (49, 1920, 128, 1920, True),    # last layer of DenseNet-201: the longest K, split over workgroups
    (784, 512, 256, 512, False),    # transition: no second batch-norm, no activation
    (8, 32, 40, 32, True),          # a single K-block, ragged rows and columns
])
def test_bn_relu_conv1x1_in_one_launch_equals_the_oracle_chain(gpu_server, rows, cin, cout, ctot, post):
    from torpor_amd.server import OP_BN_CONV1X1
    rng = np.random.default_rng(rows + cin * 3 + cout)
    X = rng.standard_normal((rows, ctot)).astype(np.float32)
    W = (rng.standard_normal((cout, cin)) / np.sqrt(cin)).astype(np.float32)
    def bn_params(c):
        return [rng.uniform(0.5, 1.5, c).astype(np.float32), rng.standard_normal(c).astype(np.float32),
                rng.standard_normal(c).astype(np.float32), rng.uniform(0.5, 2.0, c).astype(np.float32)]
    pre, pst = bn_params(cin), bn_params(cout)
    with OpSession(gpu_server, [W] + pre + pst) as t:
        x = t.act(X)
        y = t.empty(rows * cout * 4)
        t.s.launch(t.fid, OP_BN_CONV1X1, [x, *t.w[1:5], t.w[0], y, *(t.w[5:9] if post else (0, 0, 0, 0))],
                   [rows, cin, cout, ctot, 0, 1, ACT_RELU if post else ACT_NONE], [1e-5, 1e-5])
        assert t.s.last_kernel().startswith("gemm_prebn_"), t.s.last_kernel()
        got = t.read(y, (rows, cout))
        t.s.launch(t.fid, OP_BN_CONV1X1, [x, *t.w[1:5], t.w[0], y, *(t.w[5:9] if post else (0, 0, 0, 0))],
                   [rows, cin, cout, ctot, 0, 1, ACT_RELU if post else ACT_NONE], [1e-5, 1e-5])
        again = t.read(y, (rows, cout))
    xin = np.ascontiguousarray(X[:, :cin])
    a = ref.bn(xin, *pre, 1e-5, cin, nhwc=True, relu=True).reshape(rows, cin)
    if rows * cin * cout > 5e7:
        z = (a.astype(np.float64) @ W.astype(np.float64).T).astype(np.float32)
    else:
        z = ref.gemm(a, W, rows, cout, cin, cin, 1, cin, 1, cout).reshape(rows, cout)
    want = ref.bn(z, *pst, 1e-5, cout, nhwc=True, relu=True).reshape(rows, cout) if post else z
    assert_close(got, want, 5e-5, f"bn+relu+conv1x1 {rows}x{cin}->{cout}")
    assert np.array_equal(got, again), "a repeated launch must give the same bits"


def test_bn_conv1x1_without_relu_and_refusal_of_what_it_does_not_take(gpu_server):
    from torpor_amd.server import EUNSUPPORTED, OP_BN_CONV1X1, TorporError
    rng = np.random.default_rng(3)
    rows, cin, cout = 70, 64, 48
    X = rng.standard_normal((rows, cin)).astype(np.float32)
    W = (rng.standard_normal((cout, cin)) / 8).astype(np.float32)
    pre = [rng.uniform(0.5, 1.5, cin).astype(np.float32), rng.standard_normal(cin).astype(np.float32),
           rng.standard_normal(cin).astype(np.float32), rng.uniform(0.5, 2.0, cin).astype(np.float32)]
    with OpSession(gpu_server, [W] + pre) as t:
        x = t.act(X)
        y = t.empty(rows * cout * 4)
        t.s.launch(t.fid, OP_BN_CONV1X1, [x, *t.w[1:5], t.w[0], y, 0, 0, 0, 0], [rows, cin, cout, 0, 0, 0, ACT_NONE],
                   [1e-5, 1e-5])
        got = t.read(y, (rows, cout))
        a = ref.bn(X, *pre, 1e-5, cin, nhwc=True, relu=False).reshape(rows, cin)   # negative values pass
        want = ref.gemm(a, W, rows, cout, cin, cin, 1, cin, 1, cout).reshape(rows, cout)
        assert_close(got, want, 5e-5, "bn (no relu) + conv1x1")
        with pytest.raises(TorporError) as e:   # 48 input channels: not a multiple of 32
            t.s.launch(t.fid, OP_BN_CONV1X1, [x, *t.w[1:5], t.w[0], y, 0, 0, 0, 0], [rows, 48, cout, cin, 0, 1, ACT_NONE],
                       [1e-5, 1e-5])
        assert e.value.code == EUNSUPPORTED
        # like every op that fails, the refusal is reported once more at the next synchronising call (a client that
        # sends its ops in batches learns of it there)
        with pytest.raises(TorporError) as e:
            t.s.stream_synchronize(t.fid)
        assert e.value.code == EUNSUPPORTED


def test_channel_gate_on_the_operand_load_with_residual(gpu_server):
    """TP_OP_BN_CONV1X1 without beta / mean / var: x * gate[k] -> 1x1 convolution -> batch-norm + residual."""
    from torpor_amd.server import OP_BN_CONV1X1
    rng = np.random.default_rng(41)
    rows, cin, cout = 196, 480, 80
    X = rng.standard_normal((rows, cin)).astype(np.float32)
    W = (rng.standard_normal((cout, cin)) / np.sqrt(cin)).astype(np.float32)
    gate = rng.uniform(0, 1, cin).astype(np.float32)
    R = rng.standard_normal((rows, cout)).astype(np.float32)
    pst = [rng.uniform(0.5, 1.5, cout).astype(np.float32), rng.standard_normal(cout).astype(np.float32),
           rng.standard_normal(cout).astype(np.float32), rng.uniform(0.5, 2.0, cout).astype(np.float32)]
    with OpSession(gpu_server, [W] + pst) as t:
        x, g, r = t.act(X), t.act(gate), t.act(R)
        y = t.empty(rows * cout * 4)
        t.s.launch(t.fid, OP_BN_CONV1X1, [x, g, 0, 0, 0, t.w[0], y, *t.w[1:5], r], [rows, cin, cout, 0, 0, 0, ACT_NONE],
                   [0.0, 1e-5])
        assert t.s.last_kernel().startswith("gemm_prebn_"), t.s.last_kernel()
        got = t.read(y, (rows, cout))
    a = (X * gate).astype(np.float32)
    z = ref.gemm(a, W, rows, cout, cin, cin, 1, cin, 1, cout).reshape(rows, cout)
    want = ref.bn(z, *pst, 1e-5, cout, nhwc=True, relu=False).reshape(rows, cout).astype(np.float64) + R
    assert_close(got, want, 5e-5, "gate + conv1x1 + bn + residual")
