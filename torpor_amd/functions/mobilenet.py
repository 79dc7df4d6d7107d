"""MobileNetV2 (width 1.0) as a served function.

The reference serves `mobilenet_v2` from torch hub (tests/endpoint.py:30-31).  An inverted
residual block is 1x1 expand (+bn+relu6), 3x3 depthwise (+bn+relu6), 1x1 linear projection (+bn,
+identity when shapes allow); every batch-norm, activation and shortcut rides in the epilogue of
its convolution, activations are NHWC, the 3x3 stem reads the NCHW request tensor directly.
Weight names follow torchvision (`features.<i>.conv.<j>.0.weight` ...).
"""
from collections import OrderedDict

import numpy as np

from ..server import ACT_NONE, ACT_RELU6, NCHW, NHWC, OP_AVGPOOL
from .base import Function

SETTING = ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1))
BN_EPS = 1e-5


def _layers():
    """[(prefix, [(kind, cin, cout, stride)...], residual)] in torchvision's numbering."""
    out = []
    c, idx = 32, 1
    for t, cout, n, s in SETTING:
        for i in range(n):
            stride = s if i == 0 else 1
            hidden = c * t
            seq = []
            if t != 1:
                seq.append(("pw", c, hidden, 1))
            seq.append(("dw", hidden, hidden, stride))
            seq.append(("lin", hidden, cout, 1))
            out.append((f"features.{idx}.conv", seq, stride == 1 and c == cout))
            c = cout
            idx += 1
    return out, c, idx


def init_weights(seed=0, num_classes=1000):
    """torchvision's scheme: He-normal (fan_out) convolutions, batch-norm gamma=1 beta=0,
    classifier N(0, 0.01) with zero bias."""
    import torch

    g = torch.Generator().manual_seed(seed)
    w = OrderedDict()

    def conv_bn(name, cout, cin_per_group, k):
        std = (2.0 / (cout * k * k)) ** 0.5
        w[name + ".0.weight"] = torch.empty(cout, cin_per_group, k, k).normal_(0.0, std, generator=g).numpy()
        w[name + ".1.weight"] = np.ones(cout, np.float32)
        w[name + ".1.bias"] = np.zeros(cout, np.float32)
        w[name + ".1.running_mean"] = np.zeros(cout, np.float32)
        w[name + ".1.running_var"] = np.ones(cout, np.float32)

    conv_bn("features.0", 32, 3, 3)
    layers, c, idx = _layers()
    for prefix, seq, _ in layers:
        for j, (kind, cin, cout, _s) in enumerate(seq):
            conv_bn(f"{prefix}.{j}", cout, 1 if kind == "dw" else cin, 3 if kind == "dw" else 1)
    conv_bn(f"features.{idx}", 1280, c, 1)
    w["classifier.weight"] = torch.empty(num_classes, 1280).normal_(0.0, 0.01, generator=g).numpy()
    w["classifier.bias"] = np.zeros(num_classes, np.float32)
    return w


class MobileNetV2(Function):
    def __init__(self, server, fid, batch=1, weights=None, seed=0, level=1, image=224):
        super().__init__(server, fid, level)
        self.batch, self.image = batch, image
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

    def forward(self, inputs):
        (x,) = inputs
        n = self.batch
        cur, h, w = self._conv_bn(x, n, self.image, self.image, 3, 32, 3, 2, "features.0", ACT_RELU6, x_layout=NCHW)
        layers, c, idx = _layers()
        for prefix, seq, residual in layers:
            t, th, tw = cur, h, w
            for j, (kind, cin, cout, stride) in enumerate(seq):
                last = j == len(seq) - 1
                y, th, tw = self._conv_bn(t, n, th, tw, cin, cout, 3 if kind == "dw" else 1, stride, f"{prefix}.{j}",
                                          ACT_NONE if last else ACT_RELU6, groups=cin if kind == "dw" else 1,
                                          residual=cur if (last and residual) else None)
                if t is not cur:
                    self.release(t)
                t = y
            self.release(cur)
            cur, h, w = t, th, tw
        y, h, w = self._conv_bn(cur, n, h, w, c, 1280, 1, 1, f"features.{idx}", ACT_RELU6)
        self.release(cur)
        pooled = self.alloc(n * 1280 * 4)
        self.s.launch(self.fid, OP_AVGPOOL, [y.va, pooled.va], [n, h * w, 1280, NHWC])
        self.release(y)
        logits = self.alloc(n * self.num_classes * 4)
        self.s.gemm(self.fid, pooled.va, self.w["classifier.weight"], logits.va, n, self.num_classes, 1280,
                    xs_r=1280, ys_c=1280, ldc=self.num_classes, bias=self.w["classifier.bias"])
        self.release(pooled)
        return [(logits, (n, self.num_classes), np.float32)]
