"""TEST INFRASTRUCTURE ONLY - imported by tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg, never by the product.

Plain `torch.nn` ResNet (v1.5 bottleneck) and BERT encoder, run on the CPU in fp32: the
"native PyTorch path" the hot path's logits are compared with.  The reference builds its
served models from torchvision / Hugging Face packages at run time (tests/endpoint.py:16-40),
which are third-party code absent from the reference tree:
  - torchvision.models.resnet (v0.10-era, image nvcr.io/nvidia/pytorch:22.01-py3,
    dockerfiles/base.Dockerfile:18)  - not installed here; its published architecture
    (He et al. 2015 + stride on the 3x3, BN eps 1e-5, bias-free convs) is restated and pinned
    by closed-form parameter / MAC counts (tests/test_oracle_models.py).
  - transformers==4.27.1 BertModel (dockerfiles/client.Dockerfile:4-5) - a newer transformers
    is installed here; `Bert` below is pinned against it on a small config with shared weights.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

RESNET_LAYERS = {"resnet50": (3, 4, 6, 3), "resnet101": (3, 4, 23, 3), "resnet152": (3, 8, 36, 3)}


class Bottleneck(nn.Module):
    expansion = 4

    def __init__(self, inplanes, planes, stride=1, downsample=None):
        super().__init__()
        self.conv1 = nn.Conv2d(inplanes, planes, 1, bias=False)
        self.bn1 = nn.BatchNorm2d(planes)
        self.conv2 = nn.Conv2d(planes, planes, 3, stride=stride, padding=1, bias=False)
        self.bn2 = nn.BatchNorm2d(planes)
        self.conv3 = nn.Conv2d(planes, planes * 4, 1, bias=False)
        self.bn3 = nn.BatchNorm2d(planes * 4)
        self.downsample = downsample

    def forward(self, x):
        idt = x
        out = F.relu(self.bn1(self.conv1(x)))
        out = F.relu(self.bn2(self.conv2(out)))
        out = self.bn3(self.conv3(out))
        if self.downsample is not None:
            idt = self.downsample(x)
        return F.relu(out + idt)


class ResNet(nn.Module):
    def __init__(self, arch="resnet50", num_classes=1000):
        super().__init__()
        self.inplanes = 64
        self.conv1 = nn.Conv2d(3, 64, 7, stride=2, padding=3, bias=False)
        self.bn1 = nn.BatchNorm2d(64)
        blocks = RESNET_LAYERS[arch]
        self.layer1 = self._make(64, blocks[0], 1)
        self.layer2 = self._make(128, blocks[1], 2)
        self.layer3 = self._make(256, blocks[2], 2)
        self.layer4 = self._make(512, blocks[3], 2)
        self.fc = nn.Linear(2048, num_classes)

    def _make(self, planes, n, stride):
        ds = None
        if stride != 1 or self.inplanes != planes * 4:
            ds = nn.Sequential(nn.Conv2d(self.inplanes, planes * 4, 1, stride=stride, bias=False),
                               nn.BatchNorm2d(planes * 4))
        layers = [Bottleneck(self.inplanes, planes, stride, ds)]
        self.inplanes = planes * 4
        for _ in range(1, n):
            layers.append(Bottleneck(self.inplanes, planes))
        return nn.Sequential(*layers)

    def forward(self, x):
        x = F.relu(self.bn1(self.conv1(x)))
        x = F.max_pool2d(x, 3, 2, 1)
        x = self.layer4(self.layer3(self.layer2(self.layer1(x))))
        x = torch.flatten(F.adaptive_avg_pool2d(x, 1), 1)
        return self.fc(x)


class BertLayer(nn.Module):
    def __init__(self, H, A, Fd, eps):
        super().__init__()
        self.A = A
        att = nn.Module()
        att.self = nn.Module()
        att.self.query, att.self.key, att.self.value = nn.Linear(H, H), nn.Linear(H, H), nn.Linear(H, H)
        att.output = nn.Module()
        att.output.dense = nn.Linear(H, H)
        att.output.LayerNorm = nn.LayerNorm(H, eps=eps)
        self.attention = att
        self.intermediate = nn.Module()
        self.intermediate.dense = nn.Linear(H, Fd)
        self.output = nn.Module()
        self.output.dense = nn.Linear(Fd, H)
        self.output.LayerNorm = nn.LayerNorm(H, eps=eps)

    def forward(self, h, mask):
        B, S, H = h.shape
        dh = H // self.A

        def heads(t):
            return t.view(B, S, self.A, dh).permute(0, 2, 1, 3)

        sa = self.attention.self
        q, k, v = heads(sa.query(h)), heads(sa.key(h)), heads(sa.value(h))
        scores = q @ k.transpose(-1, -2) / math.sqrt(dh)
        if mask is not None:
            scores = scores + mask
        ctx = (scores.softmax(-1) @ v).permute(0, 2, 1, 3).reshape(B, S, H)
        h1 = self.attention.output.LayerNorm(self.attention.output.dense(ctx) + h)
        inter = F.gelu(self.intermediate.dense(h1))
        return self.output.LayerNorm(self.output.dense(inter) + h1)


class Bert(nn.Module):
    """Parameter names equal those of transformers.BertModel (minus buffers)."""

    def __init__(self, layers=12, hidden=768, heads=12, ffn=3072, vocab=30522, max_pos=512, type_vocab=2,
                 eps=1e-12, qa_head=False):
        super().__init__()
        emb = nn.Module()
        emb.word_embeddings = nn.Embedding(vocab, hidden)
        emb.position_embeddings = nn.Embedding(max_pos, hidden)
        emb.token_type_embeddings = nn.Embedding(type_vocab, hidden)
        emb.LayerNorm = nn.LayerNorm(hidden, eps=eps)
        self.embeddings = emb
        self.encoder = nn.Module()
        self.encoder.layer = nn.ModuleList([BertLayer(hidden, heads, ffn, eps) for _ in range(layers)])
        self.pooler = nn.Module()
        self.pooler.dense = nn.Linear(hidden, hidden)
        # transformers.BertForQuestionAnswering: span start / end logits from the last hidden state
        self.qa_outputs = nn.Linear(hidden, 2) if qa_head else None

    def forward(self, ids, token_type_ids=None, attention_mask=None):
        B, S = ids.shape
        e = self.embeddings
        tt = token_type_ids if token_type_ids is not None else torch.zeros_like(ids)
        pos = torch.arange(S).unsqueeze(0).expand(B, S)
        h = e.LayerNorm(e.word_embeddings(ids) + e.position_embeddings(pos) + e.token_type_embeddings(tt))
        mask = None
        if attention_mask is not None:
            mask = (1.0 - attention_mask[:, None, None, :].float()) * torch.finfo(torch.float32).min
        for layer in self.encoder.layer:
            h = layer(h, mask)
        if self.qa_outputs is not None:
            logits = self.qa_outputs(h)
            return logits[..., 0], logits[..., 1]
        pooled = torch.tanh(self.pooler.dense(h[:, 0]))
        return h, pooled


DENSENET_BLOCKS = {"densenet121": (6, 12, 24, 16), "densenet169": (6, 12, 32, 32), "densenet201": (6, 12, 48, 32)}


class _DenseLayer(nn.Module):
    def __init__(self, cin, growth=32, bn_size=4):
        super().__init__()
        self.norm1 = nn.BatchNorm2d(cin)
        self.conv1 = nn.Conv2d(cin, bn_size * growth, 1, bias=False)
        self.norm2 = nn.BatchNorm2d(bn_size * growth)
        self.conv2 = nn.Conv2d(bn_size * growth, growth, 3, padding=1, bias=False)

    def forward(self, x):
        return self.conv2(F.relu(self.norm2(self.conv1(F.relu(self.norm1(x))))))


class DenseNet(nn.Module):
    """Densely connected network (Huang et al. 2017) with torchvision's layer names: growth 32,
    bottleneck width 4 x growth, 64 stem channels, transitions halve channels and resolution."""

    def __init__(self, arch="densenet169", num_classes=1000, growth=32):
        super().__init__()
        f = nn.Sequential()
        f.add_module("conv0", nn.Conv2d(3, 64, 7, stride=2, padding=3, bias=False))
        f.add_module("norm0", nn.BatchNorm2d(64))
        c = 64
        blocks = DENSENET_BLOCKS[arch]
        for bi, n in enumerate(blocks):
            blk = nn.Module()
            for li in range(n):
                blk.add_module(f"denselayer{li + 1}", _DenseLayer(c + li * growth, growth))
            f.add_module(f"denseblock{bi + 1}", blk)
            c += n * growth
            if bi != len(blocks) - 1:
                tr = nn.Module()
                tr.norm = nn.BatchNorm2d(c)
                tr.conv = nn.Conv2d(c, c // 2, 1, bias=False)
                f.add_module(f"transition{bi + 1}", tr)
                c //= 2
        f.add_module("norm5", nn.BatchNorm2d(c))
        self.features = f
        self.blocks = blocks
        self.classifier = nn.Linear(c, num_classes)

    def forward(self, x):
        f = self.features
        x = F.max_pool2d(F.relu(f.norm0(f.conv0(x))), 3, 2, 1)
        for bi, n in enumerate(self.blocks):
            blk = getattr(f, f"denseblock{bi + 1}")
            for li in range(n):
                x = torch.cat([x, getattr(blk, f"denselayer{li + 1}")(x)], 1)
            if bi != len(self.blocks) - 1:
                tr = getattr(f, f"transition{bi + 1}")
                x = F.avg_pool2d(tr.conv(F.relu(tr.norm(x))), 2, 2)
        x = F.relu(f.norm5(x))
        return self.classifier(x.mean((2, 3)))


MOBILENET_V2 = ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1))


class _ConvBN(nn.Sequential):
    def __init__(self, cin, cout, k, stride=1, groups=1):
        super().__init__(nn.Conv2d(cin, cout, k, stride, k // 2, groups=groups, bias=False), nn.BatchNorm2d(cout))


class _InvertedResidual(nn.Module):
    def __init__(self, cin, cout, stride, expand):
        super().__init__()
        hidden = cin * expand
        layers = []
        if expand != 1:
            layers.append(_ConvBN(cin, hidden, 1))          # + relu6
        layers.append(_ConvBN(hidden, hidden, 3, stride, groups=hidden))  # depthwise, + relu6
        layers.append(_ConvBN(hidden, cout, 1))             # linear projection
        self.conv = nn.Sequential(*layers)
        self.residual = stride == 1 and cin == cout

    def forward(self, x):
        y = x
        for i, m in enumerate(self.conv):
            y = m(y)
            if i != len(self.conv) - 1:
                y = F.relu6(y)
        return x + y if self.residual else y


class MobileNetV2(nn.Module):
    """MobileNetV2 (Sandler et al. 2018), width 1.0: inverted residuals with linear bottlenecks."""

    def __init__(self, num_classes=1000):
        super().__init__()
        feats = [_ConvBN(3, 32, 3, 2)]
        c = 32
        for t, cout, n, s in MOBILENET_V2:
            for i in range(n):
                feats.append(_InvertedResidual(c, cout, s if i == 0 else 1, t))
                c = cout
        feats.append(_ConvBN(c, 1280, 1))
        self.features = nn.Sequential(*feats)
        self.classifier = nn.Linear(1280, num_classes)

    def forward(self, x):
        x = F.relu6(self.features[0](x))
        for m in list(self.features)[1:-1]:
            x = m(x)
        x = F.relu6(self.features[-1](x))
        return self.classifier(x.mean((2, 3)))


# (expand ratio, kernel, stride, in, out, layers) of EfficientNet-B0 (Tan & Le 2019, table 1)
EFFICIENTNET_B0 = ((1, 3, 1, 32, 16, 1), (6, 3, 2, 16, 24, 2), (6, 5, 2, 24, 40, 2), (6, 3, 2, 40, 80, 3),
                   (6, 5, 1, 80, 112, 3), (6, 5, 2, 112, 192, 4), (6, 3, 1, 192, 320, 1))


class _SqueezeExcite(nn.Module):
    def __init__(self, channels, squeeze):
        super().__init__()
        self.fc1 = nn.Conv2d(channels, squeeze, 1)
        self.fc2 = nn.Conv2d(squeeze, channels, 1)

    def forward(self, x):
        s = x.mean((2, 3), keepdim=True)
        return x * torch.sigmoid(self.fc2(F.silu(self.fc1(s))))


class _MBConv(nn.Module):
    """block.0 expand 1x1 (absent for ratio 1), then depthwise k x k, squeeze-excite (squeeze width
    = block input / 4), linear 1x1 projection; identity shortcut when stride 1 and in == out."""

    def __init__(self, cin, cout, k, stride, expand):
        super().__init__()
        hidden = cin * expand
        layers = []
        if expand != 1:
            layers.append(_ConvBN(cin, hidden, 1))
        layers.append(_ConvBN(hidden, hidden, k, stride, groups=hidden))
        layers.append(_SqueezeExcite(hidden, max(1, cin // 4)))
        layers.append(_ConvBN(hidden, cout, 1))
        self.block = nn.Sequential(*layers)
        self.residual = stride == 1 and cin == cout

    def forward(self, x):
        y = x
        for m in self.block:
            if isinstance(m, _SqueezeExcite):
                y = m(y)
            elif m is self.block[-1]:
                y = m(y)
            else:
                y = F.silu(m(y))
        return x + y if self.residual else y


class EfficientNetB0(nn.Module):
    def __init__(self, num_classes=1000):
        super().__init__()
        feats = [_ConvBN(3, 32, 3, 2)]
        for t, k, s, cin, cout, n in EFFICIENTNET_B0:
            stage = [_MBConv(cin if i == 0 else cout, cout, k, s if i == 0 else 1, t) for i in range(n)]
            feats.append(nn.Sequential(*stage))
        feats.append(_ConvBN(320, 1280, 1))
        self.features = nn.Sequential(*feats)
        self.classifier = nn.Linear(1280, num_classes)

    def forward(self, x):
        x = F.silu(self.features[0](x))
        for stage in list(self.features)[1:-1]:
            x = stage(x)
        x = F.silu(self.features[-1](x))
        return self.classifier(x.mean((2, 3)))


class _BasicConv(nn.Module):
    """conv (no bias) + batch-norm (eps 1e-3) + relu, torchvision's BasicConv2d."""

    def __init__(self, cin, cout, k, stride=1, padding=0):
        super().__init__()
        self.conv = nn.Conv2d(cin, cout, k, stride, padding, bias=False)
        self.bn = nn.BatchNorm2d(cout, eps=0.001)

    def forward(self, x):
        return F.relu(self.bn(self.conv(x)))


class _IncA(nn.Module):
    def __init__(self, cin, pool):
        super().__init__()
        self.branch1x1 = _BasicConv(cin, 64, 1)
        self.branch5x5_1 = _BasicConv(cin, 48, 1)
        self.branch5x5_2 = _BasicConv(48, 64, 5, padding=2)
        self.branch3x3dbl_1 = _BasicConv(cin, 64, 1)
        self.branch3x3dbl_2 = _BasicConv(64, 96, 3, padding=1)
        self.branch3x3dbl_3 = _BasicConv(96, 96, 3, padding=1)
        self.branch_pool = _BasicConv(cin, pool, 1)

    def forward(self, x):
        return torch.cat([self.branch1x1(x), self.branch5x5_2(self.branch5x5_1(x)),
                          self.branch3x3dbl_3(self.branch3x3dbl_2(self.branch3x3dbl_1(x))),
                          self.branch_pool(F.avg_pool2d(x, 3, 1, 1))], 1)


class _IncB(nn.Module):
    def __init__(self, cin):
        super().__init__()
        self.branch3x3 = _BasicConv(cin, 384, 3, stride=2)
        self.branch3x3dbl_1 = _BasicConv(cin, 64, 1)
        self.branch3x3dbl_2 = _BasicConv(64, 96, 3, padding=1)
        self.branch3x3dbl_3 = _BasicConv(96, 96, 3, stride=2)

    def forward(self, x):
        return torch.cat([self.branch3x3(x), self.branch3x3dbl_3(self.branch3x3dbl_2(self.branch3x3dbl_1(x))),
                          F.max_pool2d(x, 3, 2)], 1)


class _IncC(nn.Module):
    def __init__(self, cin, c7):
        super().__init__()
        self.branch1x1 = _BasicConv(cin, 192, 1)
        self.branch7x7_1 = _BasicConv(cin, c7, 1)
        self.branch7x7_2 = _BasicConv(c7, c7, (1, 7), padding=(0, 3))
        self.branch7x7_3 = _BasicConv(c7, 192, (7, 1), padding=(3, 0))
        self.branch7x7dbl_1 = _BasicConv(cin, c7, 1)
        self.branch7x7dbl_2 = _BasicConv(c7, c7, (7, 1), padding=(3, 0))
        self.branch7x7dbl_3 = _BasicConv(c7, c7, (1, 7), padding=(0, 3))
        self.branch7x7dbl_4 = _BasicConv(c7, c7, (7, 1), padding=(3, 0))
        self.branch7x7dbl_5 = _BasicConv(c7, 192, (1, 7), padding=(0, 3))
        self.branch_pool = _BasicConv(cin, 192, 1)

    def forward(self, x):
        b7 = self.branch7x7_3(self.branch7x7_2(self.branch7x7_1(x)))
        d = self.branch7x7dbl_1(x)
        for m in (self.branch7x7dbl_2, self.branch7x7dbl_3, self.branch7x7dbl_4, self.branch7x7dbl_5):
            d = m(d)
        return torch.cat([self.branch1x1(x), b7, d, self.branch_pool(F.avg_pool2d(x, 3, 1, 1))], 1)


class _IncD(nn.Module):
    def __init__(self, cin):
        super().__init__()
        self.branch3x3_1 = _BasicConv(cin, 192, 1)
        self.branch3x3_2 = _BasicConv(192, 320, 3, stride=2)
        self.branch7x7x3_1 = _BasicConv(cin, 192, 1)
        self.branch7x7x3_2 = _BasicConv(192, 192, (1, 7), padding=(0, 3))
        self.branch7x7x3_3 = _BasicConv(192, 192, (7, 1), padding=(3, 0))
        self.branch7x7x3_4 = _BasicConv(192, 192, 3, stride=2)

    def forward(self, x):
        b = self.branch7x7x3_4(self.branch7x7x3_3(self.branch7x7x3_2(self.branch7x7x3_1(x))))
        return torch.cat([self.branch3x3_2(self.branch3x3_1(x)), b, F.max_pool2d(x, 3, 2)], 1)


class _IncE(nn.Module):
    def __init__(self, cin):
        super().__init__()
        self.branch1x1 = _BasicConv(cin, 320, 1)
        self.branch3x3_1 = _BasicConv(cin, 384, 1)
        self.branch3x3_2a = _BasicConv(384, 384, (1, 3), padding=(0, 1))
        self.branch3x3_2b = _BasicConv(384, 384, (3, 1), padding=(1, 0))
        self.branch3x3dbl_1 = _BasicConv(cin, 448, 1)
        self.branch3x3dbl_2 = _BasicConv(448, 384, 3, padding=1)
        self.branch3x3dbl_3a = _BasicConv(384, 384, (1, 3), padding=(0, 1))
        self.branch3x3dbl_3b = _BasicConv(384, 384, (3, 1), padding=(1, 0))
        self.branch_pool = _BasicConv(cin, 192, 1)

    def forward(self, x):
        t = self.branch3x3_1(x)
        d = self.branch3x3dbl_2(self.branch3x3dbl_1(x))
        return torch.cat([self.branch1x1(x), self.branch3x3_2a(t), self.branch3x3_2b(t), self.branch3x3dbl_3a(d),
                          self.branch3x3dbl_3b(d), self.branch_pool(F.avg_pool2d(x, 3, 1, 1))], 1)


class InceptionV3(nn.Module):
    """Inception-v3 (Szegedy et al. 2016) as served in eval mode: torchvision's layer names, no
    auxiliary classifier, no input re-normalisation; 299x299 inputs."""

    def __init__(self, num_classes=1000):
        super().__init__()
        self.Conv2d_1a_3x3 = _BasicConv(3, 32, 3, stride=2)
        self.Conv2d_2a_3x3 = _BasicConv(32, 32, 3)
        self.Conv2d_2b_3x3 = _BasicConv(32, 64, 3, padding=1)
        self.Conv2d_3b_1x1 = _BasicConv(64, 80, 1)
        self.Conv2d_4a_3x3 = _BasicConv(80, 192, 3)
        self.Mixed_5b, self.Mixed_5c, self.Mixed_5d = _IncA(192, 32), _IncA(256, 64), _IncA(288, 64)
        self.Mixed_6a = _IncB(288)
        self.Mixed_6b, self.Mixed_6c, self.Mixed_6d, self.Mixed_6e = _IncC(768, 128), _IncC(768, 160), _IncC(768, 160), _IncC(768, 192)
        self.Mixed_7a = _IncD(768)
        self.Mixed_7b, self.Mixed_7c = _IncE(1280), _IncE(2048)
        self.fc = nn.Linear(2048, num_classes)

    def forward(self, x):
        x = self.Conv2d_2b_3x3(self.Conv2d_2a_3x3(self.Conv2d_1a_3x3(x)))
        x = F.max_pool2d(x, 3, 2)
        x = self.Conv2d_4a_3x3(self.Conv2d_3b_1x1(x))
        x = F.max_pool2d(x, 3, 2)
        for m in (self.Mixed_5b, self.Mixed_5c, self.Mixed_5d, self.Mixed_6a, self.Mixed_6b, self.Mixed_6c, self.Mixed_6d,
                  self.Mixed_6e, self.Mixed_7a, self.Mixed_7b, self.Mixed_7c):
            x = m(x)
        return self.fc(x.mean((2, 3)))


VGG16_CFG = (64, 64, "M", 128, 128, "M", 256, 256, 256, "M", 512, 512, 512, "M", 512, 512, 512, "M")


class VGG16(nn.Module):
    """VGG-16 (configuration D of Simonyan & Zisserman 2014) with torchvision's module names:
    3x3 convolutions with bias + ReLU, 2x2 max-pooling, three fully connected layers on the
    channel-major flattening of the 512 x 7 x 7 map.  Served by the reference (tests/endpoint.py:26-27)."""

    def __init__(self, num_classes=1000):
        super().__init__()
        layers, cin = [], 3
        for v in VGG16_CFG:
            if v == "M":
                layers.append(nn.MaxPool2d(2, 2))
            else:
                layers += [nn.Conv2d(cin, v, 3, padding=1), nn.ReLU(inplace=True)]
                cin = v
        self.features = nn.Sequential(*layers)
        self.classifier = nn.Sequential(nn.Linear(512 * 7 * 7, 4096), nn.ReLU(True), nn.Dropout(),
                                        nn.Linear(4096, 4096), nn.ReLU(True), nn.Dropout(), nn.Linear(4096, num_classes))

    def forward(self, x):
        x = F.adaptive_avg_pool2d(self.features(x), 7)
        return self.classifier(torch.flatten(x, 1))


class _Fire(nn.Module):
    def __init__(self, cin, squeeze, e1, e3):
        super().__init__()
        self.squeeze = nn.Conv2d(cin, squeeze, 1)
        self.expand1x1 = nn.Conv2d(squeeze, e1, 1)
        self.expand3x3 = nn.Conv2d(squeeze, e3, 3, padding=1)

    def forward(self, x):
        x = F.relu(self.squeeze(x))
        return torch.cat([F.relu(self.expand1x1(x)), F.relu(self.expand3x3(x))], 1)


class SqueezeNet11(nn.Module):
    """SqueezeNet 1.1 (Iandola et al. 2016, the lighter revision) with torchvision's module names: a 3x3
    stride-2 stem, eight fire modules (1x1 squeeze, then 1x1 and 3x3 expansions side by side), three
    3x3 stride-2 max-poolings that keep a partial last window (ceil mode), a 1x1 classifier convolution
    and a global average.  Served by the reference (tests/endpoint.py:20-21)."""

    def __init__(self, num_classes=1000):
        super().__init__()
        self.features = nn.Sequential(
            nn.Conv2d(3, 64, 3, stride=2), nn.ReLU(inplace=True), nn.MaxPool2d(3, 2, ceil_mode=True),
            _Fire(64, 16, 64, 64), _Fire(128, 16, 64, 64), nn.MaxPool2d(3, 2, ceil_mode=True),
            _Fire(128, 32, 128, 128), _Fire(256, 32, 128, 128), nn.MaxPool2d(3, 2, ceil_mode=True),
            _Fire(256, 48, 192, 192), _Fire(384, 48, 192, 192), _Fire(384, 64, 256, 256), _Fire(512, 64, 256, 256))
        self.classifier = nn.Sequential(nn.Dropout(), nn.Conv2d(512, num_classes, 1), nn.ReLU(inplace=True),
                                        nn.AdaptiveAvgPool2d(1))

    def forward(self, x):
        return torch.flatten(self.classifier(self.features(x)), 1)


def load_numpy_state(module, weights):
    """Strictly load a {name: np.ndarray} dict (BN `num_batches_tracked` buffers excepted)."""
    sd = {k: torch.from_numpy(v.copy()) for k, v in weights.items()}
    missing, unexpected = module.load_state_dict(sd, strict=False)
    missing = [m for m in missing if not m.endswith("num_batches_tracked")]
    if missing or unexpected:
        raise KeyError(f"missing={missing} unexpected={list(unexpected)}")
    return module.eval()
