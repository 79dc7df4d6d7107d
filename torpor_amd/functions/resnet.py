"""ResNet-50 / -101 / -152 (v1.5 bottleneck nets) as a served function.

The reference serves `torchvision.models.resnet*` (tests/endpoint.py:16-35); its conv, batch-norm
and elementwise layers reach the server as cuDNN calls and libtorch kernel launches.  Here the
same network is emitted as fused ops: every convolution carries its inference batch-norm and ReLU
(and the block's residual add) in its epilogue, activations are NHWC, and the 7x7 stem reads the
NCHW request tensor directly.  Weight names, shapes and initialisation follow torchvision, so a
`state_dict` of an equivalent torch module can be used as the weights.
"""
from collections import OrderedDict

import numpy as np

from ..server import ACT_NONE, ACT_RELU, NCHW, NHWC, OP_AVGPOOL, OP_MAXPOOL
from .base import Function

LAYERS = {"resnet50": (3, 4, 6, 3), "resnet101": (3, 4, 23, 3), "resnet152": (3, 8, 36, 3)}
BN_EPS = 1e-5


def init_weights(arch="resnet50", seed=0, num_classes=1000):
    """Random-init weights with torchvision's scheme: He-normal (fan_out) convolutions,
    batch-norm gamma=1 beta=0 mean=0 var=1, uniform(+-1/sqrt(fan_in)) classifier."""
    import torch

    g = torch.Generator().manual_seed(seed)
    w = OrderedDict()

    def conv(name, cout, cin, k):
        std = (2.0 / (cout * k * k)) ** 0.5
        w[name + ".weight"] = torch.empty(cout, cin, k, k).normal_(0.0, std, generator=g).numpy()

    def bn(name, c):
        w[name + ".weight"] = np.ones(c, np.float32)
        w[name + ".bias"] = np.zeros(c, np.float32)
        w[name + ".running_mean"] = np.zeros(c, np.float32)
        w[name + ".running_var"] = np.ones(c, np.float32)

    conv("conv1", 64, 3, 7)
    bn("bn1", 64)
    inplanes = 64
    for li, nblocks in enumerate(LAYERS[arch]):
        planes = 64 * (2 ** li)
        for b in range(nblocks):
            p = f"layer{li + 1}.{b}"
            stride = 2 if (b == 0 and li > 0) else 1
            conv(p + ".conv1", planes, inplanes, 1)
            bn(p + ".bn1", planes)
            conv(p + ".conv2", planes, planes, 3)
            bn(p + ".bn2", planes)
            conv(p + ".conv3", planes * 4, planes, 1)
            bn(p + ".bn3", planes * 4)
            if b == 0 and (stride != 1 or inplanes != planes * 4):
                conv(p + ".downsample.0", planes * 4, inplanes, 1)
                bn(p + ".downsample.1", planes * 4)
            inplanes = planes * 4
    bound = 1.0 / (inplanes ** 0.5)
    w["fc.weight"] = (torch.rand(num_classes, inplanes, generator=g) * 2 - 1).mul_(bound).numpy()
    w["fc.bias"] = (torch.rand(num_classes, generator=g) * 2 - 1).mul_(bound).numpy()
    return w


class ResNet(Function):
    def __init__(self, server, fid, arch="resnet50", batch=1, weights=None, seed=0, level=1, image=224):
        super().__init__(server, fid, level)
        self.arch, self.batch, self.image = arch, batch, image
        self._weights = weights if weights is not None else init_weights(arch, seed)
        self.num_classes = self._weights["fc.weight"].shape[0]

    def weights(self):
        return OrderedDict((k, np.ascontiguousarray(v, dtype=np.float32)) for k, v in self._weights.items()
                           if not k.endswith("num_batches_tracked"))

    def input_specs(self):
        return [((self.batch, 3, self.image, self.image), np.float32)]

    def _bn(self, name):
        return (self.w[name + ".weight"], self.w[name + ".bias"], self.w[name + ".running_mean"],
                self.w[name + ".running_var"])

    def _conv(self, x, n, h, w, cin, cout, k, stride, pad, wname, bnname, act, residual=None, x_layout=NHWC):
        ho = (h + 2 * pad - k) // stride + 1
        wo = (w + 2 * pad - k) // stride + 1
        y = self.alloc(n * ho * wo * cout * 4)
        self.s.conv(self.fid, x.va, self.w[wname + ".weight"], y.va, n, h, w, cin, cout, k, k, stride=stride,
                    pad=pad, x_layout=x_layout, y_layout=NHWC, bn=self._bn(bnname), bn_eps=BN_EPS,
                    residual=residual.va if residual is not None else 0, act=act)
        return y, ho, wo

    def forward(self, inputs):
        (x,) = inputs
        n = self.batch
        t, h, w = self._conv(x, n, self.image, self.image, 3, 64, 7, 2, 3, "conv1", "bn1", ACT_RELU, x_layout=NCHW)
        ho, wo = (h + 2 - 3) // 2 + 1, (w + 2 - 3) // 2 + 1
        p = self.alloc(n * ho * wo * 64 * 4)
        self.s.launch(self.fid, OP_MAXPOOL, [t.va, p.va], [n, h, w, 64, 3, 2, 1, NHWC])
        self.release(t)
        cur, h, w, inplanes = p, ho, wo, 64
        for li, nblocks in enumerate(LAYERS[self.arch]):
            planes = 64 * (2 ** li)
            for b in range(nblocks):
                pre = f"layer{li + 1}.{b}"
                stride = 2 if (b == 0 and li > 0) else 1
                t1, _, _ = self._conv(cur, n, h, w, inplanes, planes, 1, 1, 0, pre + ".conv1", pre + ".bn1", ACT_RELU)
                t2, h2, w2 = self._conv(t1, n, h, w, planes, planes, 3, stride, 1, pre + ".conv2", pre + ".bn2",
                                        ACT_RELU)
                self.release(t1)
                if (pre + ".downsample.0.weight") in self.w:
                    idt, _, _ = self._conv(cur, n, h, w, inplanes, planes * 4, 1, stride, 0, pre + ".downsample.0",
                                           pre + ".downsample.1", ACT_NONE)
                    self.release(cur)
                else:
                    idt = cur
                out, _, _ = self._conv(t2, n, h2, w2, planes, planes * 4, 1, 1, 0, pre + ".conv3", pre + ".bn3",
                                       ACT_RELU, residual=idt)
                self.release(t2)
                self.release(idt)
                cur, h, w, inplanes = out, h2, w2, planes * 4
        pooled = self.alloc(n * inplanes * 4)
        self.s.launch(self.fid, OP_AVGPOOL, [cur.va, pooled.va], [n, h * w, inplanes, NHWC])
        self.release(cur)
        logits = self.alloc(n * self.num_classes * 4)
        self.s.gemm(self.fid, pooled.va, self.w["fc.weight"], logits.va, n, self.num_classes, inplanes,
                    xs_r=inplanes, ys_c=inplanes, ldc=self.num_classes, bias=self.w["fc.bias"])
        self.release(pooled)
        return [(logits, (n, self.num_classes), np.float32)]
