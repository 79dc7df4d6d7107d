"""DenseNet-121 / -169 / -201 as a served function.

The reference serves `torchvision.models.densenet169` / `densenet201` (tests/endpoint.py:20-23).
Each dense layer is bn-relu-conv1x1-bn-relu-conv3x3 whose 32 new channels are concatenated to its
input.  Here a dense block owns one NHWC buffer as wide as the block's final channel count: a
layer's 1x1 convolution reads the first `cin` channels of it (input pitch), applies the first
batch-norm + ReLU to them as it loads them and carries the second batch-norm + ReLU in its
epilogue (one launch, TP_OP_BN_CONV1X1; two -- batch-norm into a dense temporary, then the
convolution -- where the library has no kernel for the fused form), and the 3x3 convolution
writes its 32 channels straight into the block buffer at channel offset `cin` (output pitch), so
nothing is ever concatenated by copying.  Transitions average-pool directly into the next
block's buffer.  Weight names follow torchvision.
"""
from collections import OrderedDict

import numpy as np

from ..server import ACT_NONE, ACT_RELU, NCHW, NHWC, OP_AVGPOOL, OP_AVGPOOL2D, OP_BN_CONV1X1, OP_COPY2D, OP_MAXPOOL
from .base import Function

BLOCKS = {"densenet121": (6, 12, 24, 16), "densenet169": (6, 12, 32, 32), "densenet201": (6, 12, 48, 32)}
GROWTH, BN_SIZE, BN_EPS = 32, 4, 1e-5


def init_weights(arch="densenet169", seed=0, num_classes=1000):
    """torchvision's scheme: He-normal convolutions, batch-norm gamma=1 beta=0, classifier bias 0."""
    import torch

    g = torch.Generator().manual_seed(seed)
    w = OrderedDict()

    def conv(name, cout, cin, k):
        std = (2.0 / (cin * k * k)) ** 0.5
        w[name + ".weight"] = torch.empty(cout, cin, k, k).normal_(0.0, std, generator=g).numpy()

    def bn(name, c):
        w[name + ".weight"] = np.ones(c, np.float32)
        w[name + ".bias"] = np.zeros(c, np.float32)
        w[name + ".running_mean"] = np.zeros(c, np.float32)
        w[name + ".running_var"] = np.ones(c, np.float32)

    conv("features.conv0", 64, 3, 7)
    bn("features.norm0", 64)
    c = 64
    blocks = BLOCKS[arch]
    for bi, n in enumerate(blocks):
        for li in range(n):
            p = f"features.denseblock{bi + 1}.denselayer{li + 1}"
            bn(p + ".norm1", c + li * GROWTH)
            conv(p + ".conv1", BN_SIZE * GROWTH, c + li * GROWTH, 1)
            bn(p + ".norm2", BN_SIZE * GROWTH)
            conv(p + ".conv2", GROWTH, BN_SIZE * GROWTH, 3)
        c += n * GROWTH
        if bi != len(blocks) - 1:
            p = f"features.transition{bi + 1}"
            bn(p + ".norm", c)
            conv(p + ".conv", c // 2, c, 1)
            c //= 2
    bn("features.norm5", c)
    bound = 1.0 / (c ** 0.5)
    w["classifier.weight"] = (torch.rand(num_classes, c, generator=g) * 2 - 1).mul_(bound).numpy()
    w["classifier.bias"] = np.zeros(num_classes, np.float32)
    return w


class DenseNet(Function):
    def __init__(self, server, fid, arch="densenet169", batch=1, weights=None, seed=0, level=1, image=224, fused=None):
        super().__init__(server, fid, level)
        self.arch, self.batch, self.image = arch, batch, image
        self._weights = weights if weights is not None else init_weights(arch, seed)
        self.num_classes = self._weights["classifier.weight"].shape[0]
        self._fused = fused   # False: always batch-norm and convolution as two calls (for comparison)

    def weights(self):
        return OrderedDict((k, np.ascontiguousarray(v, dtype=np.float32)) for k, v in self._weights.items()
                           if not k.endswith("num_batches_tracked"))

    def input_specs(self):
        return [((self.batch, 3, self.image, self.image), np.float32)]

    def _bn(self, name):
        return (self.w[name + ".weight"], self.w[name + ".bias"], self.w[name + ".running_mean"],
                self.w[name + ".running_var"])

    def _bn_relu(self, x_va, rows, c, name, x_pitch=0):
        y = self.alloc(rows * c * 4)
        self.s.bn(self.fid, x_va, y.va, *self._bn(name), BN_EPS, rows, c, relu=True, x_pitch=x_pitch)
        return y

    def _bn_relu_conv1x1(self, x_va, n, h, w, cin, cout, pre, weight, post=None, x_pitch=0):
        """relu(bn_pre(x)) -> 1x1 convolution -> (bn_post + relu when `post` is given); returns the output block."""
        rows = n * h * w
        y = self.alloc(rows * cout * 4)
        # what TP_OP_BN_CONV1X1 takes (include/torpor_amd.h): cin a multiple of 32 up to 2048, 16-byte aligned rows
        if self._fused is not False and cin % 32 == 0 and cin <= 2048 and x_pitch % 4 == 0 and x_va % 16 == 0:
            self.s.launch(self.fid, OP_BN_CONV1X1,
                          [x_va, *self._bn(pre), self.w[weight], y.va, *(self._bn(post) if post else (0, 0, 0, 0))],
                          [rows, cin, cout, x_pitch, 0, 1, ACT_RELU if post else ACT_NONE], [BN_EPS, BN_EPS])
            return y
        t = self._bn_relu(x_va, rows, cin, pre, x_pitch=x_pitch)
        if post:
            self.s.conv(self.fid, t.va, self.w[weight], y.va, n, h, w, cin, cout, 1, 1, bn=self._bn(post),
                        bn_eps=BN_EPS, act=ACT_RELU)
        else:
            self.s.conv(self.fid, t.va, self.w[weight], y.va, n, h, w, cin, cout, 1, 1)
        self.release(t)
        return y

    def forward(self, inputs):
        (x,) = inputs
        n, s = self.batch, self.s
        h = w = (self.image + 6 - 7) // 2 + 1
        stem = self.alloc(n * h * w * 64 * 4)
        s.conv(self.fid, x.va, self.w["features.conv0.weight"], stem.va, n, self.image, self.image, 3, 64, 7, 7,
               stride=2, pad=3, x_layout=NCHW, y_layout=NHWC, bn=self._bn("features.norm0"), bn_eps=BN_EPS,
               act=ACT_RELU)
        ho, wo = (h + 2 - 3) // 2 + 1, (w + 2 - 3) // 2 + 1
        pooled = self.alloc(n * ho * wo * 64 * 4)
        s.launch(self.fid, OP_MAXPOOL, [stem.va, pooled.va], [n, h, w, 64, 3, 2, 1, NHWC])
        self.release(stem)
        h, w, c = ho, wo, 64
        blocks = BLOCKS[self.arch]
        buf = None
        for bi, nl in enumerate(blocks):
            ctot = c + nl * GROWTH
            rows = n * h * w
            if buf is None:
                buf = self.alloc(rows * ctot * 4)
                s.launch(self.fid, OP_COPY2D, [pooled.va, buf.va], [rows, c, c, ctot])
                self.release(pooled)
            for li in range(nl):
                p = f"features.denseblock{bi + 1}.denselayer{li + 1}"
                cin = c + li * GROWTH
                t2 = self._bn_relu_conv1x1(buf.va, n, h, w, cin, BN_SIZE * GROWTH, p + ".norm1", p + ".conv1.weight",
                                           post=p + ".norm2", x_pitch=ctot)
                # the 32 new channels land next to the ones the layer read
                s.conv(self.fid, t2.va, self.w[p + ".conv2.weight"], buf.va + cin * 4, n, h, w, BN_SIZE * GROWTH,
                       GROWTH, 3, 3, stride=1, pad=1, y_pitch=ctot, act=ACT_NONE)
                self.release(t2)
            c = ctot
            if bi != len(blocks) - 1:
                p = f"features.transition{bi + 1}"
                t2 = self._bn_relu_conv1x1(buf.va, n, h, w, c, c // 2, p + ".norm", p + ".conv.weight")
                self.release(buf)
                c //= 2
                nh, nw = h // 2, w // 2
                nxt_tot = c + blocks[bi + 1] * GROWTH
                buf = self.alloc(n * nh * nw * nxt_tot * 4)
                s.launch(self.fid, OP_AVGPOOL2D, [t2.va, buf.va], [n, h, w, c, 2, 2, 0, nxt_tot])
                self.release(t2)
                h, w = nh, nw
        rows = n * h * w
        t1 = self._bn_relu(buf.va, rows, c, "features.norm5")
        self.release(buf)
        pooled = self.alloc(n * c * 4)
        s.launch(self.fid, OP_AVGPOOL, [t1.va, pooled.va], [n, h * w, c, NHWC])
        self.release(t1)
        logits = self.alloc(n * self.num_classes * 4)
        s.gemm(self.fid, pooled.va, self.w["classifier.weight"], logits.va, n, self.num_classes, c, xs_r=c, ys_c=c,
               ldc=self.num_classes, bias=self.w["classifier.bias"])
        self.release(pooled)
        return [(logits, (n, self.num_classes), np.float32)]
