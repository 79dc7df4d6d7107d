"""SqueezeNet 1.1 as a served function (the reference serves `torchvision.models.squeezenet1_1`,
tests/endpoint.py:20-21).

A fire module squeezes with a 1x1 convolution and expands with a 1x1 and a 3x3 convolution whose
outputs are concatenated; here both expansions write their channels straight into the two halves of
the module's output (output pitch), so nothing is copied.  All convolutions carry their bias and ReLU
in the epilogue.  The three max-poolings are 3x3 / stride 2 in ceil mode; the image side is restricted
to sizes where no window is partial (224 is one), where ceil and floor mode agree.  Weight names follow
torchvision."""
from collections import OrderedDict

import numpy as np

from ..server import ACT_RELU, NCHW, NHWC, OP_AVGPOOL, OP_MAXPOOL
from .base import Function

FIRES = ((64, 16, 64, 64), (128, 16, 64, 64), "M", (128, 32, 128, 128), (256, 32, 128, 128), "M",
         (256, 48, 192, 192), (384, 48, 192, 192), (384, 64, 256, 256), (512, 64, 256, 256))


def init_weights(seed=0, num_classes=1000):
    """torchvision's scheme: He-uniform convolutions, N(0, 0.01) for the classifier convolution, zero biases."""
    import torch

    g = torch.Generator().manual_seed(seed)
    w = OrderedDict()

    def conv(name, cout, cin, k, final=False):
        if final:
            t = torch.empty(cout, cin, k, k).normal_(0.0, 0.01, generator=g)
        else:
            bound = (6.0 / (cin * k * k)) ** 0.5
            t = (torch.rand(cout, cin, k, k, generator=g) * 2 - 1) * bound
        w[name + ".weight"] = t.numpy()
        w[name + ".bias"] = np.zeros(cout, np.float32)

    conv("features.0", 64, 3, 3)
    idx = 3
    for f in FIRES:
        if f == "M":
            idx += 1
            continue
        cin, sq, e1, e3 = f
        conv(f"features.{idx}.squeeze", sq, cin, 1)
        conv(f"features.{idx}.expand1x1", e1, sq, 1)
        conv(f"features.{idx}.expand3x3", e3, sq, 3)
        idx += 1
    conv("classifier.1", num_classes, 512, 1, final=True)
    return w


def _pool_out(h):
    if (h - 3) % 2:
        raise ValueError("image side leaves a partial pooling window (ceil mode is not reproduced)")
    return (h - 3) // 2 + 1


class SqueezeNet11(Function):
    def __init__(self, server, fid, batch=1, weights=None, seed=0, level=1, image=224):
        super().__init__(server, fid, level)
        self.batch, self.image = batch, image
        self._weights = weights if weights is not None else init_weights(seed)
        self.num_classes = self._weights["classifier.1.weight"].shape[0]
        h = (image - 3) // 2 + 1
        for _ in range(3):   # refuse unsupported sizes at construction
            h = _pool_out(h)

    def weights(self):
        return OrderedDict((k, np.ascontiguousarray(v, dtype=np.float32)) for k, v in self._weights.items())

    def input_specs(self):
        return [((self.batch, 3, self.image, self.image), np.float32)]

    def _conv(self, x_va, y_va, n, h, w, cin, cout, k, name, stride=1, pad=0, x_layout=NHWC, y_pitch=0):
        self.s.conv(self.fid, x_va, self.w[name + ".weight"], y_va, n, h, w, cin, cout, k, k, stride=stride, pad=pad,
                    x_layout=x_layout, y_layout=NHWC, y_pitch=y_pitch, bias=self.w[name + ".bias"], act=ACT_RELU)

    def _maxpool(self, cur, n, h, w, c):
        ho, wo = _pool_out(h), _pool_out(w)
        y = self.alloc(n * ho * wo * c * 4)
        self.s.launch(self.fid, OP_MAXPOOL, [cur.va, y.va], [n, h, w, c, 3, 2, 0, NHWC])
        self.release(cur)
        return y, ho, wo

    def forward(self, inputs):
        (x,) = inputs
        n = self.batch
        h = w = (self.image - 3) // 2 + 1
        cur = self.alloc(n * h * w * 64 * 4)
        self._conv(x.va, cur.va, n, self.image, self.image, 3, 64, 3, "features.0", stride=2, x_layout=NCHW)
        cur, h, w = self._maxpool(cur, n, h, w, 64)
        c, idx = 64, 3
        for f in FIRES:
            if f == "M":
                cur, h, w = self._maxpool(cur, n, h, w, c)
                idx += 1
                continue
            cin, sq, e1, e3 = f
            assert cin == c
            p = f"features.{idx}"
            t = self.alloc(n * h * w * sq * 4)
            self._conv(cur.va, t.va, n, h, w, cin, sq, 1, p + ".squeeze")
            self.release(cur)
            out = self.alloc(n * h * w * (e1 + e3) * 4)
            self._conv(t.va, out.va, n, h, w, sq, e1, 1, p + ".expand1x1", y_pitch=e1 + e3)
            self._conv(t.va, out.va + e1 * 4, n, h, w, sq, e3, 3, p + ".expand3x3", pad=1, y_pitch=e1 + e3)
            self.release(t)
            cur, c = out, e1 + e3
            idx += 1
        y = self.alloc(n * h * w * self.num_classes * 4)
        self._conv(cur.va, y.va, n, h, w, c, self.num_classes, 1, "classifier.1")
        self.release(cur)
        logits = self.alloc(n * self.num_classes * 4)
        self.s.launch(self.fid, OP_AVGPOOL, [y.va, logits.va], [n, h * w, self.num_classes, NHWC])
        self.release(y)
        return [(logits, (n, self.num_classes), np.float32)]
