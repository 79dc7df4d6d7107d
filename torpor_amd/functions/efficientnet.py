"""EfficientNet-B0 as a served function.

The reference serves `torchvision.models.efficientnet_b0` (tests/endpoint.py:34-35).  An MBConv block
is 1x1 expand (+bn+silu), k x k depthwise (+bn+silu), squeeze-and-excitation, 1x1 linear projection
(+bn, +identity when shapes allow).  Batch-norm, SiLU and the shortcut ride in convolution
epilogues; the squeeze-and-excitation branch is a global average pool and two small GEMMs whose
epilogues apply bias + SiLU and bias + sigmoid; the gate is applied by the projection itself as it loads
its input (one image, channel counts the fused kernel takes) or by a gating pass over the activations.
Weight names follow torchvision (`features.<stage>.<layer>.block.<j>...`).
"""
from collections import OrderedDict

import numpy as np

from ..server import ACT_NONE, ACT_SIGMOID, ACT_SILU, NCHW, NHWC, OP_AVGPOOL, OP_BN_CONV1X1, OP_SCALE_CHANNELS
from .base import Function

# (expand ratio, kernel, stride, in, out, layers)
STAGES = ((1, 3, 1, 32, 16, 1), (6, 3, 2, 16, 24, 2), (6, 5, 2, 24, 40, 2), (6, 3, 2, 40, 80, 3),
          (6, 5, 1, 80, 112, 3), (6, 5, 2, 112, 192, 4), (6, 3, 1, 192, 320, 1))
BN_EPS = 1e-5


def _blocks():
    """[(prefix, cin, cout, kernel, stride, expand)] in torchvision's numbering."""
    out = []
    for si, (t, k, s, cin, cout, n) in enumerate(STAGES):
        for i in range(n):
            out.append((f"features.{si + 1}.{i}.block", cin if i == 0 else cout, cout, k, s if i == 0 else 1, t))
    return out


def init_weights(seed=0, num_classes=1000):
    """torchvision's scheme: He-normal (fan_out) convolutions with zero bias, batch-norm gamma=1
    beta=0, classifier uniform(+-1/sqrt(out)).  The squeeze-excite biases get small random values
    instead of zeros so that they influence the output."""
    import torch

    g = torch.Generator().manual_seed(seed)
    w = OrderedDict()

    def conv(name, cout, cin_per_group, k, bias=False):
        std = (2.0 / (cout * k * k)) ** 0.5
        w[name + ".weight"] = torch.empty(cout, cin_per_group, k, k).normal_(0.0, std, generator=g).numpy()
        if bias:
            w[name + ".bias"] = torch.empty(cout).normal_(0.0, 0.1, generator=g).numpy()

    def bn(name, c):
        w[name + ".weight"] = np.ones(c, np.float32)
        w[name + ".bias"] = np.zeros(c, np.float32)
        w[name + ".running_mean"] = np.zeros(c, np.float32)
        w[name + ".running_var"] = np.ones(c, np.float32)

    conv("features.0.0", 32, 3, 3)
    bn("features.0.1", 32)
    for prefix, cin, cout, k, stride, t in _blocks():
        hidden, j = cin * t, 0
        if t != 1:
            conv(f"{prefix}.{j}.0", hidden, cin, 1)
            bn(f"{prefix}.{j}.1", hidden)
            j += 1
        conv(f"{prefix}.{j}.0", hidden, 1, k)
        bn(f"{prefix}.{j}.1", hidden)
        j += 1
        sq = max(1, cin // 4)
        conv(f"{prefix}.{j}.fc1", sq, hidden, 1, bias=True)
        conv(f"{prefix}.{j}.fc2", hidden, sq, 1, bias=True)
        j += 1
        conv(f"{prefix}.{j}.0", cout, hidden, 1)
        bn(f"{prefix}.{j}.1", cout)
    conv("features.8.0", 1280, 320, 1)
    bn("features.8.1", 1280)
    bound = 1.0 / (num_classes ** 0.5)
    w["classifier.weight"] = (torch.rand(num_classes, 1280, generator=g) * 2 - 1).mul_(bound).numpy()
    w["classifier.bias"] = np.zeros(num_classes, np.float32)
    return w


class EfficientNetB0(Function):
    def __init__(self, server, fid, batch=1, weights=None, seed=0, level=1, image=224, fused=None):
        super().__init__(server, fid, level)
        self.batch, self.image = batch, image
        self._fused = fused   # False: the channel gate always as a pass of its own (for comparison)
        self._weights = weights if weights is not None else init_weights(seed)
        self.num_classes = self._weights["classifier.weight"].shape[0]

    def weights(self):
        return OrderedDict((k, np.ascontiguousarray(v, dtype=np.float32)) for k, v in self._weights.items()
                           if not k.endswith("num_batches_tracked"))

    def input_specs(self):
        return [((self.batch, 3, self.image, self.image), np.float32)]

    def _conv_bn(self, x, n, h, w, cin, cout, k, stride, name, act, groups=1, residual=None, x_layout=NHWC):
        pad = k // 2
        ho, wo = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
        y = self.alloc(n * ho * wo * cout * 4)
        bn = tuple(self.w[f"{name}.1.{f}"] for f in ("weight", "bias", "running_mean", "running_var"))
        self.s.conv(self.fid, x.va, self.w[name + ".0.weight"], y.va, n, h, w, cin, cout, k, k, stride=stride, pad=pad,
                    x_layout=x_layout, y_layout=NHWC, groups=groups, bn=bn, bn_eps=BN_EPS,
                    residual=residual.va if residual is not None else 0, act=act)
        return y, ho, wo

    def _squeeze_excite(self, x, n, hw, c, sq, name):
        pooled = self.alloc(n * c * 4)
        self.s.launch(self.fid, OP_AVGPOOL, [x.va, pooled.va], [n, hw, c, NHWC])
        mid = self.alloc(n * sq * 4)
        self.s.gemm(self.fid, pooled.va, self.w[name + ".fc1.weight"], mid.va, n, sq, c, xs_r=c, ys_c=c, ldc=sq,
                    bias=self.w[name + ".fc1.bias"], act=ACT_SILU)
        self.release(pooled)
        gate = self.alloc(n * c * 4)
        self.s.gemm(self.fid, mid.va, self.w[name + ".fc2.weight"], gate.va, n, c, sq, xs_r=sq, ys_c=sq, ldc=c,
                    bias=self.w[name + ".fc2.bias"], act=ACT_SIGMOID)
        self.release(mid)
        return gate

    def _gate_and_project(self, x, gate, n, h, w, c, cout, name, residual):
        """y = bn(conv1x1(x * gate)) (+ residual).  One image and a channel count the library's fused kernel
        takes (TP_OP_BN_CONV1X1 with a plain per-channel scale on the operand load): one launch; otherwise the
        gating pass and the convolution."""
        rows = n * h * w
        if n == 1 and c % 32 == 0 and c <= 2048 and self._fused is not False:
            y = self.alloc(rows * cout * 4)
            bn = tuple(self.w[f"{name}.1.{f}"] for f in ("weight", "bias", "running_mean", "running_var"))
            self.s.launch(self.fid, OP_BN_CONV1X1,
                          [x.va, gate.va, 0, 0, 0, self.w[name + ".0.weight"], y.va, *bn,
                           residual.va if residual is not None else 0],
                          [rows, c, cout, 0, 0, 0, ACT_NONE], [0.0, BN_EPS])
            return y
        g = self.alloc(rows * c * 4)
        self.s.launch(self.fid, OP_SCALE_CHANNELS, [x.va, gate.va, g.va], [n, h * w, c])
        y, _, _ = self._conv_bn(g, n, h, w, c, cout, 1, 1, name, ACT_NONE, residual=residual)
        self.release(g)
        return y

    def forward(self, inputs):
        (x,) = inputs
        n = self.batch
        cur, h, w = self._conv_bn(x, n, self.image, self.image, 3, 32, 3, 2, "features.0", ACT_SILU, x_layout=NCHW)
        for prefix, cin, cout, k, stride, t in _blocks():
            hidden, j = cin * t, 0
            y = cur
            if t != 1:
                y, _, _ = self._conv_bn(cur, n, h, w, cin, hidden, 1, 1, f"{prefix}.{j}", ACT_SILU)
                j += 1
            d, h2, w2 = self._conv_bn(y, n, h, w, hidden, hidden, k, stride, f"{prefix}.{j}", ACT_SILU, groups=hidden)
            if y is not cur:
                self.release(y)
            j += 1
            gate = self._squeeze_excite(d, n, h2 * w2, hidden, max(1, cin // 4), f"{prefix}.{j}")
            j += 1
            out = self._gate_and_project(d, gate, n, h2, w2, hidden, cout, f"{prefix}.{j}",
                                         cur if (stride == 1 and cin == cout) else None)
            self.release(gate)
            self.release(d)
            self.release(cur)
            cur, h, w = out, h2, w2
        y, h, w = self._conv_bn(cur, n, h, w, 320, 1280, 1, 1, "features.8", ACT_SILU)
        self.release(cur)
        pooled = self.alloc(n * 1280 * 4)
        self.s.launch(self.fid, OP_AVGPOOL, [y.va, pooled.va], [n, h * w, 1280, NHWC])
        self.release(y)
        logits = self.alloc(n * self.num_classes * 4)
        self.s.gemm(self.fid, pooled.va, self.w["classifier.weight"], logits.va, n, self.num_classes, 1280,
                    xs_r=1280, ys_c=1280, ldc=self.num_classes, bias=self.w["classifier.bias"])
        self.release(pooled)
        return [(logits, (n, self.num_classes), np.float32)]
