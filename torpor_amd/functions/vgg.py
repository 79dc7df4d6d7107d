"""VGG-16 as a served function (the reference serves `torchvision.models.vgg16`, tests/endpoint.py:26-27).

Thirteen 3x3 convolutions with bias and ReLU in the convolution's epilogue, five 2x2 max-poolings, and
three fully connected layers.  Activations are NHWC; torchvision flattens the last 512 x 7 x 7 map channel
first, so that map is turned to NCHW once (25088 floats per image) before the first fully connected layer
and the uploaded weights are used as they are.  Weight names follow torchvision."""
from collections import OrderedDict

import numpy as np

from ..server import ACT_NONE, ACT_RELU, NCHW, NHWC, OP_AVGPOOL2D, OP_MAXPOOL, OP_NHWC_TO_NCHW
from .base import Function

CFG = (64, 64, "M", 128, 128, "M", 256, 256, 256, "M", 512, 512, 512, "M", 512, 512, 512, "M")


def init_weights(seed=0, num_classes=1000):
    """torchvision's scheme: He-normal (fan-out) convolutions with zero bias, N(0, 0.01) linear layers."""
    import torch

    g = torch.Generator().manual_seed(seed)
    w = OrderedDict()
    cin, idx = 3, 0
    for v in CFG:
        if v == "M":
            idx += 1
            continue
        std = (2.0 / (v * 9)) ** 0.5
        w[f"features.{idx}.weight"] = torch.empty(v, cin, 3, 3).normal_(0.0, std, generator=g).numpy()
        w[f"features.{idx}.bias"] = np.zeros(v, np.float32)
        cin = v
        idx += 2
    for i, (o, k) in zip((0, 3, 6), ((4096, 25088), (4096, 4096), (num_classes, 4096))):
        w[f"classifier.{i}.weight"] = torch.empty(o, k).normal_(0.0, 0.01, generator=g).numpy()
        w[f"classifier.{i}.bias"] = np.zeros(o, np.float32)
    return w


class VGG16(Function):
    def __init__(self, server, fid, batch=1, weights=None, seed=0, level=1, image=224):
        super().__init__(server, fid, level)
        if image % 32:
            raise ValueError("image side must be a multiple of 32")
        self.batch, self.image = batch, image
        self._weights = weights if weights is not None else init_weights(seed)
        self.num_classes = self._weights["classifier.6.weight"].shape[0]

    def weights(self):
        return OrderedDict((k, np.ascontiguousarray(v, dtype=np.float32)) for k, v in self._weights.items())

    def input_specs(self):
        return [((self.batch, 3, self.image, self.image), np.float32)]

    def forward(self, inputs):
        (cur,) = inputs
        n, s = self.batch, self.s
        h = w = self.image
        cin, idx, layout = 3, 0, NCHW
        for v in CFG:
            if v == "M":
                y = self.alloc(n * (h // 2) * (w // 2) * cin * 4)
                s.launch(self.fid, OP_MAXPOOL, [cur.va, y.va], [n, h, w, cin, 2, 2, 0, NHWC])
                self.release(cur)
                cur, h, w = y, h // 2, w // 2
                idx += 1
                continue
            y = self.alloc(n * h * w * v * 4)
            s.conv(self.fid, cur.va, self.w[f"features.{idx}.weight"], y.va, n, h, w, cin, v, 3, 3, stride=1, pad=1,
                   x_layout=layout, y_layout=NHWC, bias=self.w[f"features.{idx}.bias"], act=ACT_RELU)
            if layout == NHWC:
                self.release(cur)
            cur, cin, layout = y, v, NHWC
            idx += 2
        if h != 7:   # adaptive average pooling to 7 x 7 (the identity at 224 x 224)
            k = h // 7
            y = self.alloc(n * 49 * cin * 4)
            s.launch(self.fid, OP_AVGPOOL2D, [cur.va, y.va], [n, h, w, cin, k, k, 0, 0])
            self.release(cur)
            cur, h, w = y, 7, 7
        flat = self.alloc(n * cin * 49 * 4)   # channel-major, as torch.flatten sees the NCHW map
        s.launch(self.fid, OP_NHWC_TO_NCHW, [cur.va, flat.va], [n, cin, 7, 7])
        self.release(cur)
        cur, k = flat, cin * 49
        for i, act in ((0, ACT_RELU), (3, ACT_RELU), (6, ACT_NONE)):
            o = self._weights[f"classifier.{i}.weight"].shape[0]
            y = self.alloc(n * o * 4)
            s.gemm(self.fid, cur.va, self.w[f"classifier.{i}.weight"], y.va, n, o, k, xs_r=k, ys_c=k, ldc=o,
                   bias=self.w[f"classifier.{i}.bias"], act=act)
            self.release(cur)
            cur, k = y, o
        return [(cur, (n, self.num_classes), np.float32)]
