"""Inception-v3 as a served function (eval mode, no auxiliary classifier, 299x299 inputs).

The reference serves `torchvision.models.inception_v3` (tests/endpoint.py:32-33).  Every
BasicConv2d (conv + batch-norm eps 1e-3 + ReLU) is one fused convolution; the branches of a
Mixed block write their last convolution (or max-pool) straight into their channel slice of the
block's output buffer (output pitch), so the concatenations cost nothing.  The asymmetric 1x7 /
7x1 / 1x3 / 3x1 convolutions run on the general convolution kernel.  Weight names follow
torchvision.
"""
from collections import OrderedDict

import numpy as np

from ..server import ACT_RELU, NCHW, NHWC, OP_AVGPOOL, OP_AVGPOOL2D, OP_MAXPOOL
from .base import Function

BN_EPS = 1e-3


def _spec():
    """[(name, cin, cout, (kh, kw), stride, (ph, pw))] of every BasicConv2d, in torchvision's order."""
    L = []

    def c(name, cin, cout, k, stride=1, pad=0):
        k = (k, k) if isinstance(k, int) else k
        pad = (pad, pad) if isinstance(pad, int) else pad
        L.append((name, cin, cout, k, stride, pad))

    c("Conv2d_1a_3x3", 3, 32, 3, 2)
    c("Conv2d_2a_3x3", 32, 32, 3)
    c("Conv2d_2b_3x3", 32, 64, 3, 1, 1)
    c("Conv2d_3b_1x1", 64, 80, 1)
    c("Conv2d_4a_3x3", 80, 192, 3)
    for name, cin, pool in (("Mixed_5b", 192, 32), ("Mixed_5c", 256, 64), ("Mixed_5d", 288, 64)):
        c(name + ".branch1x1", cin, 64, 1)
        c(name + ".branch5x5_1", cin, 48, 1)
        c(name + ".branch5x5_2", 48, 64, 5, 1, 2)
        c(name + ".branch3x3dbl_1", cin, 64, 1)
        c(name + ".branch3x3dbl_2", 64, 96, 3, 1, 1)
        c(name + ".branch3x3dbl_3", 96, 96, 3, 1, 1)
        c(name + ".branch_pool", cin, pool, 1)
    c("Mixed_6a.branch3x3", 288, 384, 3, 2)
    c("Mixed_6a.branch3x3dbl_1", 288, 64, 1)
    c("Mixed_6a.branch3x3dbl_2", 64, 96, 3, 1, 1)
    c("Mixed_6a.branch3x3dbl_3", 96, 96, 3, 2)
    for name, c7 in (("Mixed_6b", 128), ("Mixed_6c", 160), ("Mixed_6d", 160), ("Mixed_6e", 192)):
        c(name + ".branch1x1", 768, 192, 1)
        c(name + ".branch7x7_1", 768, c7, 1)
        c(name + ".branch7x7_2", c7, c7, (1, 7), 1, (0, 3))
        c(name + ".branch7x7_3", c7, 192, (7, 1), 1, (3, 0))
        c(name + ".branch7x7dbl_1", 768, c7, 1)
        c(name + ".branch7x7dbl_2", c7, c7, (7, 1), 1, (3, 0))
        c(name + ".branch7x7dbl_3", c7, c7, (1, 7), 1, (0, 3))
        c(name + ".branch7x7dbl_4", c7, c7, (7, 1), 1, (3, 0))
        c(name + ".branch7x7dbl_5", c7, 192, (1, 7), 1, (0, 3))
        c(name + ".branch_pool", 768, 192, 1)
    c("Mixed_7a.branch3x3_1", 768, 192, 1)
    c("Mixed_7a.branch3x3_2", 192, 320, 3, 2)
    c("Mixed_7a.branch7x7x3_1", 768, 192, 1)
    c("Mixed_7a.branch7x7x3_2", 192, 192, (1, 7), 1, (0, 3))
    c("Mixed_7a.branch7x7x3_3", 192, 192, (7, 1), 1, (3, 0))
    c("Mixed_7a.branch7x7x3_4", 192, 192, 3, 2)
    for name, cin in (("Mixed_7b", 1280), ("Mixed_7c", 2048)):
        c(name + ".branch1x1", cin, 320, 1)
        c(name + ".branch3x3_1", cin, 384, 1)
        c(name + ".branch3x3_2a", 384, 384, (1, 3), 1, (0, 1))
        c(name + ".branch3x3_2b", 384, 384, (3, 1), 1, (1, 0))
        c(name + ".branch3x3dbl_1", cin, 448, 1)
        c(name + ".branch3x3dbl_2", 448, 384, 3, 1, 1)
        c(name + ".branch3x3dbl_3a", 384, 384, (1, 3), 1, (0, 1))
        c(name + ".branch3x3dbl_3b", 384, 384, (3, 1), 1, (1, 0))
        c(name + ".branch_pool", cin, 192, 1)
    return L


SPEC = OrderedDict((s[0], s[1:]) for s in _spec())


def init_weights(seed=0, num_classes=1000):
    """He-normal (fan_in) convolutions, batch-norm gamma=1 beta=0 mean=0 var=1, N(0, 1/fan_in)
    classifier.  (torchvision draws every weight from a truncated normal of std 0.1, which relies on
    training-time batch statistics; with the identity batch-norm of a fresh model that would
    overflow fp32 after a few layers.)"""
    import torch

    g = torch.Generator().manual_seed(seed)
    w = OrderedDict()
    for name, (cin, cout, k, _s, _p) in SPEC.items():
        std = (2.0 / (cin * k[0] * k[1])) ** 0.5
        w[name + ".conv.weight"] = torch.empty(cout, cin, k[0], k[1]).normal_(0.0, std, generator=g).numpy()
        w[name + ".bn.weight"] = np.ones(cout, np.float32)
        w[name + ".bn.bias"] = np.zeros(cout, np.float32)
        w[name + ".bn.running_mean"] = np.zeros(cout, np.float32)
        w[name + ".bn.running_var"] = np.ones(cout, np.float32)
    w["fc.weight"] = torch.empty(num_classes, 2048).normal_(0.0, 2048 ** -0.5, generator=g).numpy()
    w["fc.bias"] = np.zeros(num_classes, np.float32)
    return w


class InceptionV3(Function):
    def __init__(self, server, fid, batch=1, weights=None, seed=0, level=1, image=299):
        super().__init__(server, fid, level)
        self.batch, self.image = batch, image
        self._weights = weights if weights is not None else init_weights(seed)
        self.num_classes = self._weights["fc.weight"].shape[0]

    def weights(self):
        return OrderedDict((k, np.ascontiguousarray(v, dtype=np.float32)) for k, v in self._weights.items()
                           if not k.endswith("num_batches_tracked"))

    def input_specs(self):
        return [((self.batch, 3, self.image, self.image), np.float32)]

    # one BasicConv2d; writes into `out_va` with pixel pitch `pitch` when given, else into a new buffer
    def _bc(self, name, x_va, h, w, out_va=None, pitch=0, x_layout=NHWC):
        cin, cout, k, stride, pad = SPEC[name]
        ho, wo = (h + 2 * pad[0] - k[0]) // stride + 1, (w + 2 * pad[1] - k[1]) // stride + 1
        buf = None
        if out_va is None:
            buf = self.alloc(self.batch * ho * wo * cout * 4)
            out_va = buf.va
        bn = tuple(self.w[f"{name}.bn.{f}"] for f in ("weight", "bias", "running_mean", "running_var"))
        self.s.conv(self.fid, x_va, self.w[name + ".conv.weight"], out_va, self.batch, h, w, cin, cout, k[0], k[1],
                    stride=stride, pad=pad, x_layout=x_layout, y_layout=NHWC, y_pitch=pitch, bn=bn, bn_eps=BN_EPS,
                    act=ACT_RELU)
        return buf, ho, wo

    def _chain(self, names, x_va, h, w, out_va, pitch):
        """names[:-1] into temporaries, names[-1] into the output slice."""
        t, va = None, x_va
        for nm in names[:-1]:
            nt, h, w = self._bc(nm, va, h, w)
            if t is not None:
                self.release(t)
            t, va = nt, nt.va
        self._bc(names[-1], va, h, w, out_va, pitch)
        if t is not None:
            self.release(t)

    def _pool_branch(self, name, x, h, w, cin, out_va, pitch):
        p = self.alloc(self.batch * h * w * cin * 4)
        self.s.launch(self.fid, OP_AVGPOOL2D, [x.va, p.va], [self.batch, h, w, cin, 3, 1, 1, 0])
        self._bc(name, p.va, h, w, out_va, pitch)
        self.release(p)

    def _mixed(self, name, x, h, w, cin):
        n, kind = self.batch, name[:7]
        branches = []   # (kind, conv names, width)
        if name in ("Mixed_5b", "Mixed_5c", "Mixed_5d"):
            pool = SPEC[name + ".branch_pool"][1]
            branches = [("c", ["branch1x1"], 64), ("c", ["branch5x5_1", "branch5x5_2"], 64),
                        ("c", ["branch3x3dbl_1", "branch3x3dbl_2", "branch3x3dbl_3"], 96), ("avg", ["branch_pool"], pool)]
            ho, wo = h, w
        elif name == "Mixed_6a":
            branches = [("c", ["branch3x3"], 384), ("c", ["branch3x3dbl_1", "branch3x3dbl_2", "branch3x3dbl_3"], 96),
                        ("max", [], cin)]
            ho, wo = (h - 3) // 2 + 1, (w - 3) // 2 + 1
        elif kind == "Mixed_6":
            branches = [("c", ["branch1x1"], 192), ("c", ["branch7x7_1", "branch7x7_2", "branch7x7_3"], 192),
                        ("c", ["branch7x7dbl_%d" % i for i in range(1, 6)], 192), ("avg", ["branch_pool"], 192)]
            ho, wo = h, w
        elif name == "Mixed_7a":
            branches = [("c", ["branch3x3_1", "branch3x3_2"], 320),
                        ("c", ["branch7x7x3_%d" % i for i in range(1, 5)], 192), ("max", [], cin)]
            ho, wo = (h - 3) // 2 + 1, (w - 3) // 2 + 1
        else:   # Mixed_7b / 7c: two branches fork at their end
            branches = [("c", ["branch1x1"], 320), ("fork", ["branch3x3_1"], 768, ["branch3x3_2a", "branch3x3_2b"]),
                        ("fork", ["branch3x3dbl_1", "branch3x3dbl_2"], 768, ["branch3x3dbl_3a", "branch3x3dbl_3b"]),
                        ("avg", ["branch_pool"], 192)]
            ho, wo = h, w
        ctot = sum(b[2] for b in branches)
        out = self.alloc(n * ho * wo * ctot * 4)
        off = 0
        for b in branches:
            va = out.va + off * 4
            if b[0] == "c":
                self._chain([f"{name}.{c}" for c in b[1]], x.va, h, w, va, ctot)
            elif b[0] == "avg":
                self._pool_branch(f"{name}.{b[1][0]}", x, h, w, cin, va, ctot)
            elif b[0] == "max":
                self.s.launch(self.fid, OP_MAXPOOL, [x.va, va], [n, h, w, cin, 3, 2, 0, NHWC, ctot])
            else:
                t, tva, th, tw = None, x.va, h, w
                for c in b[1]:
                    nt, th, tw = self._bc(f"{name}.{c}", tva, th, tw)
                    if t is not None:
                        self.release(t)
                    t, tva = nt, nt.va
                self._bc(f"{name}.{b[3][0]}", tva, th, tw, va, ctot)
                self._bc(f"{name}.{b[3][1]}", tva, th, tw, va + 384 * 4, ctot)
                self.release(t)
            off += b[2]
        return out, ho, wo, ctot

    def forward(self, inputs):
        (x,) = inputs
        n = self.batch
        t, h, w = self._bc("Conv2d_1a_3x3", x.va, self.image, self.image, x_layout=NCHW)
        for nm in ("Conv2d_2a_3x3", "Conv2d_2b_3x3"):
            nt, h, w = self._bc(nm, t.va, h, w)
            self.release(t)
            t = nt
        c = 64
        for nm in (None, "Conv2d_3b_1x1", "Conv2d_4a_3x3", None):
            if nm is None:
                ho, wo = (h - 3) // 2 + 1, (w - 3) // 2 + 1
                nt = self.alloc(n * ho * wo * c * 4)
                self.s.launch(self.fid, OP_MAXPOOL, [t.va, nt.va], [n, h, w, c, 3, 2, 0, NHWC])
                h, w = ho, wo
            else:
                nt, h, w = self._bc(nm, t.va, h, w)
                c = SPEC[nm][1]
            self.release(t)
            t = nt
        for nm in ("Mixed_5b", "Mixed_5c", "Mixed_5d", "Mixed_6a", "Mixed_6b", "Mixed_6c", "Mixed_6d", "Mixed_6e",
                   "Mixed_7a", "Mixed_7b", "Mixed_7c"):
            nt, h, w, c = self._mixed(nm, t, h, w, c)
            self.release(t)
            t = nt
        pooled = self.alloc(n * c * 4)
        self.s.launch(self.fid, OP_AVGPOOL, [t.va, pooled.va], [n, h * w, c, NHWC])
        self.release(t)
        logits = self.alloc(n * self.num_classes * 4)
        self.s.gemm(self.fid, pooled.va, self.w["fc.weight"], logits.va, n, self.num_classes, c, xs_r=c, ys_c=c,
                    ldc=self.num_classes, bias=self.w["fc.bias"])
        self.release(pooled)
        return [(logits, (n, self.num_classes), np.float32)]
