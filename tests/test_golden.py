"""Known-answer vectors (tests/golden/vectors.npz, written by tests/golden/make_vectors.py from
numpy / torch float64 library routines): the C oracle must reproduce them on the CPU, and the HIP
kernels must reproduce them on the GPU through the C-ABI."""
import os

import numpy as np
import pytest

from oracle import ops as ref
from tests.harness import assert_close

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz"))
TOL = 2e-5


def test_oracle_reproduces_the_golden_vectors():
    X, W = V["gemm_x"], V["gemm_w"]
    z = ref.gemm(X, W, 37, 50, 72, 72, 1, 72, 1, 50).reshape(37, 50) + V["gemm_b"]
    assert_close(z, V["gemm_y"], 1e-6, "gemm")
    assert_close(ref.gelu(V["gemm_y"]), V["gemm_gelu"], 2e-6, "gelu")
    y = ref.conv2d(V["conv_x"], V["conv_w"], (2, 2), (1, 1), x_nhwc=True, y_nhwc=True)
    assert_close(y, V["conv_y"], 1e-6, "conv3x3")
    yb = ref.bn(y, V["conv_g"], V["conv_b"], V["conv_mu"], V["conv_var"], 1e-5, 24, nhwc=True, relu=True)
    assert_close(yb, V["conv_bn_relu"], 2e-6, "conv+bn+relu")
    assert_close(ref.conv2d(V["conv_x"], V["conv1_w"], (2, 2), (0, 0), x_nhwc=True, y_nhwc=True), V["conv1_y"], 1e-6, "1x1")
    assert_close(ref.depthwise_conv2d(V["conv_x"], V["dw_w"], (1, 1), (1, 1)), V["dw_y"], 1e-6, "depthwise")
    ys1 = ref.conv2d(V["conv_x"], V["conv_s1_w"], (1, 1), (1, 1), x_nhwc=True, y_nhwc=True).astype(np.float64)
    assert_close(np.maximum(ys1 + V["conv_s1_res"], 0), V["conv_s1_y"], 1e-6, "conv3x3 stride 1 + residual + relu")
    assert_close(ref.layernorm(V["ln_x"], V["ln_r"], V["ln_g"], V["ln_b"], 1e-12), V["ln_y"], 2e-6, "layernorm")
    assert_close(ref.softmax(V["sm_x"], V["sm_mask"], 0.125, 1), V["sm_y"], 2e-6, "softmax")
    assert_close(ref.attention(V["att_q"], V["att_k"], V["att_v"], V["att_mask"], 0.125), V["att_y"], 2e-6, "attention")
    np.testing.assert_array_equal(ref.maxpool(V["conv_x"], 3, 2, 1, nhwc=True), V["maxpool_y"])
    assert_close(ref.avgpool(V["conv_x"], nhwc=True), V["avgpool_y"], 2e-6, "avgpool")
    assert_close(ref.embedding(V["emb_ids"], V["emb_tids"], V["emb_word"], V["emb_pos"], V["emb_typ"], 9), V["emb_y"],
                 1e-6, "embedding")


@pytest.mark.gpu
def test_kernels_reproduce_the_golden_vectors(gpu_server):
    from tests.harness import OpSession
    from torpor_amd.server import (ACT_GELU, ACT_RELU, NHWC, OP_ATTENTION, OP_AVGPOOL, OP_EMBEDDING, OP_LAYERNORM,
                                   OP_MAXPOOL, OP_SOFTMAX)
    weights = [V[k] for k in ("gemm_w", "gemm_b", "conv_w", "conv_g", "conv_b", "conv_mu", "conv_var", "conv1_w", "dw_w",
                              "ln_g", "ln_b", "emb_word", "emb_pos", "emb_typ")]
    with OpSession(gpu_server, weights) as t:
        s, f, w = t.s, t.fid, t.w
        x = t.act(V["gemm_x"])
        c = t.empty(37 * 50 * 4)
        s.gemm(f, x, w[0], c, 37, 50, 72, xs_r=72, ys_c=72, ldc=50, bias=w[1])
        assert_close(t.read(c, (37, 50)), V["gemm_y"], TOL, "gemm")
        s.gemm(f, x, w[0], c, 37, 50, 72, xs_r=72, ys_c=72, ldc=50, bias=w[1], act=ACT_GELU)
        assert_close(t.read(c, (37, 50)), V["gemm_gelu"], TOL, "gemm+gelu")

        cx = t.act(V["conv_x"])
        cy = t.empty(V["conv_y"].nbytes)
        s.conv(f, cx, w[2], cy, 2, 9, 8, 16, 24, 3, 3, stride=2, pad=1)
        assert_close(t.read(cy, V["conv_y"].shape), V["conv_y"], TOL, "conv3x3")
        s.conv(f, cx, w[2], cy, 2, 9, 8, 16, 24, 3, 3, stride=2, pad=1, bn=tuple(w[3:7]), bn_eps=1e-5, act=ACT_RELU)
        assert_close(t.read(cy, V["conv_y"].shape), V["conv_bn_relu"], TOL, "conv+bn+relu")
        c1 = t.empty(V["conv1_y"].nbytes)
        s.conv(f, cx, w[7], c1, 2, 9, 8, 16, 12, 1, 1, stride=2, pad=0)
        assert_close(t.read(c1, V["conv1_y"].shape), V["conv1_y"], TOL, "1x1 stride 2")
        dy = t.empty(V["dw_y"].nbytes)
        s.conv(f, cx, w[8], dy, 2, 9, 8, 16, 16, 3, 3, stride=1, pad=1, groups=16)
        assert_close(t.read(dy, V["dw_y"].shape), V["dw_y"], TOL, "depthwise")

        lx, lr = t.act(V["ln_x"]), t.act(V["ln_r"])
        ly = t.empty(V["ln_y"].nbytes)
        s.launch(f, OP_LAYERNORM, [lx, lr, w[9], w[10], ly], [11, 96], [1e-12])
        assert_close(t.read(ly, (11, 96)), V["ln_y"], TOL, "layernorm")

        sx, sm = t.act(V["sm_x"]), t.act(V["sm_mask"])
        sy = t.empty(V["sm_y"].nbytes)
        s.launch(f, OP_SOFTMAX, [sx, sm, sy], [6, 40, 1], [0.125])
        assert_close(t.read(sy, (6, 40)), V["sm_y"], 2e-6, "softmax")

        q, k, v, am = (t.act(V[n]) for n in ("att_q", "att_k", "att_v", "att_mask"))
        ay = t.empty(V["att_y"].nbytes)
        s.launch(f, OP_ATTENTION, [q, k, v, am, ay], [2, 2, 40, 64, 128, 128, 128, 128], [0.125])
        assert_close(t.read(ay, V["att_y"].shape), V["att_y"], TOL, "attention")

        my = t.empty(V["maxpool_y"].nbytes)
        s.launch(f, OP_MAXPOOL, [cx, my], [2, 9, 8, 16, 3, 2, 1, NHWC])
        np.testing.assert_array_equal(t.read(my, V["maxpool_y"].shape), V["maxpool_y"])
        ay2 = t.empty(V["avgpool_y"].nbytes)
        s.launch(f, OP_AVGPOOL, [cx, ay2], [2, 72, 16, NHWC])
        assert_close(t.read(ay2, (2, 16)), V["avgpool_y"], 2e-6, "avgpool")

        ids, tids = t.act(V["emb_ids"]), t.act(V["emb_tids"])
        ey = t.empty(V["emb_y"].nbytes)
        s.launch(f, OP_EMBEDDING, [ids, tids, w[11], w[12], w[13], ey], [18, 9, 24, 30, 2])
        assert_close(t.read(ey, (18, 24)), V["emb_y"], 1e-6, "embedding")


@pytest.mark.gpu
@pytest.mark.parametrize("path", ["winograd", "direct"])
def test_stride_1_3x3_convolution_reproduces_the_golden_vectors_on_both_paths(gpu_server, monkeypatch, path):
    """16 -> 32 channels, stride 1, residual + ReLU: the Winograd path (sent down it below its size bound) and the
    direct kernels against the same float64 library result."""
    from tests.harness import OpSession
    from torpor_amd.server import ACT_RELU
    monkeypatch.setenv("TORPOR_WINOGRAD", "1" if path == "winograd" else "0")
    monkeypatch.setenv("TORPOR_WINO_MIN_GFLOP", "0")
    with OpSession(gpu_server, [V["conv_s1_w"]]) as t:
        cx, cr = t.act(V["conv_x"]), t.act(V["conv_s1_res"])
        cy = t.empty(V["conv_s1_y"].nbytes)
        t.s.conv(t.fid, cx, t.w[0], cy, 2, 9, 8, 16, 32, 3, 3, stride=1, pad=1, residual=cr, act=ACT_RELU)
        assert t.s.last_kernel().startswith("conv3x3_wino" if path == "winograd" else "conv3x3_fast"), t.s.last_kernel()
        assert_close(t.read(cy, V["conv_s1_y"].shape), V["conv_s1_y"], TOL, f"conv3x3 stride 1 ({path})")
