"""Pins the whole-model oracle (oracle/models.py).  ResNet: closed-form parameter and MAC counts
of the published v1.5 bottleneck architecture (torchvision is not installed).  BERT: the
installed `transformers` BertModel on a small in-code config with shared weights (third-party
code, no download).  Product-side weight generators must load strictly into these modules."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import models as om
from torpor_amd.functions import bert as pbert
from torpor_amd.functions import resnet as presnet


def _macs(model, x):
    total = [0]

    def hook(mod, inp, out):
        if isinstance(mod, torch.nn.Conv2d):
            total[0] += out.numel() * (mod.in_channels // mod.groups) * mod.kernel_size[0] * mod.kernel_size[1]
        elif isinstance(mod, torch.nn.Linear):
            total[0] += out.numel() * mod.in_features

    hs = [m.register_forward_hook(hook) for m in model.modules()]
    with torch.no_grad():
        y = model(x)
    for h in hs:
        h.remove()
    return total[0], y


def _closed_form_macs(blocks):
    """MACs of a v1.5 bottleneck ResNet on one 224x224 image, from the architecture table alone."""
    total = 112 * 112 * 64 * 3 * 49                      # 7x7/2 stem
    hw, inplanes = 56, 64
    for stage, n in enumerate(blocks):
        planes = 64 * 2 ** stage
        for b in range(n):
            stride = 2 if (b == 0 and stage > 0) else 1
            out_hw = hw // stride
            total += hw * hw * planes * inplanes                     # 1x1 reduce (input resolution)
            total += out_hw * out_hw * planes * planes * 9           # 3x3, carries the stride
            total += out_hw * out_hw * planes * 4 * planes           # 1x1 expand
            if b == 0:
                total += out_hw * out_hw * planes * 4 * inplanes     # projection shortcut
            hw, inplanes = out_hw, planes * 4
    return total + 2048 * 1000


@pytest.mark.parametrize("arch,params,gmacs", [("resnet50", 25557032, 4.089), ("resnet101", 44549160, 7.801),
                                               ("resnet152", 60192808, 11.514)])
def test_resnet_counts(arch, params, gmacs):
    """25,557,032 / 44,549,160 / 60,192,808 parameters and 4.089 / 7.801 / 11.514 GMAC per 224x224
    image are the published figures for ResNet-50 / -101 / -152 (v1.5 moves the stride, not the counts)."""
    model = om.ResNet(arch).eval()
    assert sum(p.numel() for p in model.parameters()) == params
    m, y = _macs(model, torch.zeros(1, 3, 224, 224))
    assert y.shape == (1, 1000)
    assert m == _closed_form_macs(om.RESNET_LAYERS[arch]), m
    assert round(m / 1e9, 3) == gmacs
    n_weight_tensors = len(list(model.parameters()))
    n_bn_buffers = sum(1 for k in model.state_dict() if "running" in k)
    assert (n_weight_tensors, n_bn_buffers) == {"resnet50": (161, 106), "resnet101": (314, 208), "resnet152": (467, 310)}[arch]


def test_resnet_stride_is_on_the_3x3():
    model = om.ResNet("resnet50")
    b = model.layer2[0]
    assert b.conv1.stride == (1, 1) and b.conv2.stride == (2, 2) and b.downsample[0].stride == (2, 2)
    assert model.bn1.eps == 1e-5 and model.conv1.bias is None


@pytest.mark.parametrize("arch", ["resnet50", "resnet152"])
def test_product_resnet_weights_load_strictly(arch):
    w = presnet.init_weights(arch, seed=0)
    om.load_numpy_state(om.ResNet(arch), w)
    # He-normal, fan_out: std = sqrt(2 / (cout * k * k))
    c = w["layer1.0.conv2.weight"]
    assert abs(c.std() - (2.0 / (64 * 9)) ** 0.5) < 2e-3
    assert np.array_equal(presnet.init_weights(arch, seed=0)["fc.weight"], w["fc.weight"])      # deterministic
    assert not np.array_equal(presnet.init_weights(arch, seed=1)["fc.weight"], w["fc.weight"])


@pytest.mark.parametrize("arch,params", [("bert-base", 109482240), ("bert-large", 335141888)])
def test_bert_param_counts(arch, params):
    cfg = pbert.CONFIGS[arch]
    with torch.device("meta"):
        model = om.Bert(**cfg)
    assert sum(p.numel() for p in model.parameters()) == params
    assert len(list(model.parameters())) == {"bert-base": 199, "bert-large": 391}[arch]


def test_bert_matches_transformers():
    transformers = pytest.importorskip("transformers")
    cfg = transformers.BertConfig(vocab_size=97, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
                                  intermediate_size=128, max_position_embeddings=40, type_vocab_size=2,
                                  hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0)
    torch.manual_seed(0)
    hf = transformers.BertModel(cfg).eval()
    assert cfg.layer_norm_eps == 1e-12 and cfg.hidden_act == "gelu"
    mine = om.Bert(layers=2, hidden=64, heads=4, ffn=128, vocab=97, max_pos=40, type_vocab=2)
    sd = {k: v for k, v in hf.state_dict().items() if k in mine.state_dict()}
    assert set(sd) == set(mine.state_dict()), set(mine.state_dict()) - set(sd)
    mine.load_state_dict(sd)
    mine.eval()
    ids = torch.randint(0, 97, (3, 17))
    tt = torch.randint(0, 2, (3, 17))
    am = torch.ones(3, 17, dtype=torch.long)
    am[1, 11:] = 0
    with torch.no_grad():
        ref = hf(input_ids=ids, token_type_ids=tt, attention_mask=am)
        h, pooled = mine(ids, tt, am)
    assert torch.allclose(h, ref.last_hidden_state, atol=2e-5, rtol=1e-4)
    assert torch.allclose(pooled, ref.pooler_output, atol=2e-5, rtol=1e-4)
    with torch.no_grad():   # defaults: token types 0, no mask
        ref0 = hf(input_ids=ids)
        h0, p0 = mine(ids)
    assert torch.allclose(h0, ref0.last_hidden_state, atol=2e-5, rtol=1e-4)


def test_product_bert_weights_load_strictly():
    cfg = dict(layers=2, hidden=64, heads=4, ffn=128)
    w = pbert.init_weights(seed=0, vocab=97, max_pos=40, cfg=cfg)
    om.load_numpy_state(om.Bert(vocab=97, max_pos=40, **cfg), w)
    assert abs(w["encoder.layer.0.intermediate.dense.weight"].std() - 0.02) < 2e-3


def test_bert_qa_head_matches_transformers():
    """The question-answering variant the reference serves (tests/endpoint.py:36-40,
    BertForQuestionAnswering called with input ids and token type ids): span logits of the oracle
    against the installed transformers implementation with shared weights."""
    transformers = pytest.importorskip("transformers")
    cfg = transformers.BertConfig(vocab_size=97, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
                                  intermediate_size=128, max_position_embeddings=40, type_vocab_size=2,
                                  hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0)
    torch.manual_seed(1)
    hf = transformers.BertForQuestionAnswering(cfg).eval()
    mine = om.Bert(layers=2, hidden=64, heads=4, ffn=128, vocab=97, max_pos=40, type_vocab=2, qa_head=True)
    want = {k[len("bert."):] if k.startswith("bert.") else k: v for k, v in hf.state_dict().items()}
    sd = {k: v for k, v in want.items() if k in mine.state_dict()}
    # the transformers model has no pooler; the oracle's stays at its initial value and is unused
    assert set(mine.state_dict()) - set(sd) == {"pooler.dense.weight", "pooler.dense.bias"}
    mine.load_state_dict(sd, strict=False)
    mine.eval()
    ids = torch.randint(0, 97, (2, 19))
    tt = torch.randint(0, 2, (2, 19))
    am = torch.ones(2, 19, dtype=torch.long)
    am[0, 13:] = 0
    with torch.no_grad():
        ref = hf(input_ids=ids, token_type_ids=tt, attention_mask=am)
        start, end = mine(ids, tt, am)
    assert torch.allclose(start, ref.start_logits, atol=2e-5, rtol=1e-4)
    assert torch.allclose(end, ref.end_logits, atol=2e-5, rtol=1e-4)
    # product-side weight generator loads strictly, and its mask helper equals the oracle's convention
    w = pbert.init_weights(cfg=dict(layers=2, hidden=64, heads=4, ffn=128), vocab=97, max_pos=40, qa_head=True)
    om.load_numpy_state(om.Bert(layers=2, hidden=64, heads=4, ffn=128, vocab=97, max_pos=40, qa_head=True), w)
    add = pbert.Bert.additive_mask(am.numpy())
    assert add.dtype == np.float32 and (add[0, :13] == 0).all() and (add[0, 13:] == np.finfo(np.float32).min).all()


@pytest.mark.parametrize("arch,params,gmacs", [("densenet121", 7978856, 2.834), ("densenet169", 14149480, 3.360),
                                               ("densenet201", 20013928, 4.291)])
def test_densenet_counts(arch, params, gmacs):
    """Published parameter counts (7,978,856 / 14,149,480 / 20,013,928) and multiply-accumulates per
    224x224 image (2.83 / 3.36 / 4.29 G) of DenseNet-121 / -169 / -201, and the channel bookkeeping
    of the dense blocks (each layer sees 32 more channels; transitions halve them)."""
    model = om.DenseNet(arch).eval()
    assert sum(p.numel() for p in model.parameters()) == params
    m, y = _macs(model, torch.zeros(1, 3, 224, 224))
    assert y.shape == (1, 1000)
    assert round(m / 1e9, 3) == gmacs
    c = 64
    for bi, n in enumerate(om.DENSENET_BLOCKS[arch]):
        blk = getattr(model.features, f"denseblock{bi + 1}")
        for li in range(n):
            assert getattr(blk, f"denselayer{li + 1}").conv1.in_channels == c + 32 * li
        c += 32 * n
        if bi != 3:
            assert getattr(model.features, f"transition{bi + 1}").conv.out_channels == c // 2
            c //= 2
    assert model.classifier.in_features == c == {"densenet121": 1024, "densenet169": 1664, "densenet201": 1920}[arch]


def test_densenet_layer_matches_functional_definition():
    """One dense layer is conv3x3(relu(bn(conv1x1(relu(bn(x)))))) concatenated to its input."""
    torch.manual_seed(3)
    model = om.DenseNet("densenet121").eval()
    layer = model.features.denseblock1.denselayer1
    for bn in (layer.norm1, layer.norm2):
        bn.running_mean.normal_()
        bn.running_var.uniform_(0.5, 2.0)
    x = torch.randn(2, 64, 9, 9)
    with torch.no_grad():
        t = F.batch_norm(x, layer.norm1.running_mean, layer.norm1.running_var, layer.norm1.weight, layer.norm1.bias,
                         False, 0.0, 1e-5).relu()
        t = F.conv2d(t, layer.conv1.weight)
        t = F.batch_norm(t, layer.norm2.running_mean, layer.norm2.running_var, layer.norm2.weight, layer.norm2.bias,
                         False, 0.0, 1e-5).relu()
        want = F.conv2d(t, layer.conv2.weight, padding=1)
        assert torch.allclose(layer(x), want, atol=1e-6)


def test_mobilenet_v2_counts():
    """3,504,872 parameters and 300.8 M multiply-accumulates per 224x224 image (published), 17
    inverted-residual blocks of which 10 have an identity shortcut."""
    model = om.MobileNetV2().eval()
    assert sum(p.numel() for p in model.parameters()) == 3504872
    m, y = _macs(model, torch.zeros(1, 3, 224, 224))
    assert y.shape == (1, 1000)
    assert round(m / 1e6, 1) == 300.8
    blocks = [b for b in model.features if isinstance(b, om._InvertedResidual)]
    assert len(blocks) == 17 and sum(b.residual for b in blocks) == 10
    dw = [c for b in blocks for c in b.modules() if isinstance(c, torch.nn.Conv2d) and c.groups > 1]
    assert len(dw) == 17 and all(c.groups == c.in_channels == c.out_channels for c in dw)


def test_efficientnet_b0_counts():
    """5,288,548 parameters and 0.39 G multiply-accumulates per 224x224 image (published); 16 MBConv
    blocks, squeeze width = block input / 4, 9 identity shortcuts; the product-side weight generator
    loads strictly."""
    model = om.EfficientNetB0().eval()
    assert sum(p.numel() for p in model.parameters()) == 5288548
    m, y = _macs(model, torch.zeros(1, 3, 224, 224))
    assert y.shape == (1, 1000)
    assert round(m / 1e9, 2) == 0.39
    blocks = [b for b in model.modules() if isinstance(b, om._MBConv)]
    assert len(blocks) == 16 and sum(b.residual for b in blocks) == 9
    se = [s_ for s_ in model.modules() if isinstance(s_, om._SqueezeExcite)]
    assert [s_.fc1.out_channels for s_ in se][:4] == [8, 4, 6, 6]
    from torpor_amd.functions import efficientnet as peff
    om.load_numpy_state(om.EfficientNetB0(), peff.init_weights())


def test_squeeze_excite_matches_functional_definition():
    torch.manual_seed(5)
    se = om._SqueezeExcite(12, 3).eval()
    x = torch.randn(2, 12, 5, 4)
    with torch.no_grad():
        s_ = x.mean((2, 3))
        g = torch.sigmoid(F.linear(F.silu(F.linear(s_, se.fc1.weight.flatten(1), se.fc1.bias)), se.fc2.weight.flatten(1),
                                   se.fc2.bias))
        assert torch.allclose(se(x), x * g[:, :, None, None], atol=1e-6)


def test_inception_v3_counts():
    """23,834,568 parameters without the auxiliary classifier (27,161,264 published with it, whose own
    share is 3,326,696) and 5.71 G multiply-accumulates per 299x299 image; 94 conv + batch-norm pairs;
    output widths of the Mixed blocks 256, 288, 288, 768 x5, 1280, 2048, 2048."""
    model = om.InceptionV3().eval()
    assert sum(p.numel() for p in model.parameters()) == 23834568 == 27161264 - 3326696
    m, y = _macs(model, torch.zeros(1, 3, 299, 299))
    assert y.shape == (1, 1000) and round(m / 1e9, 2) == 5.71
    assert sum(1 for c in model.modules() if isinstance(c, torch.nn.Conv2d)) == 94
    widths, x = [], torch.zeros(1, 192, 35, 35)
    with torch.no_grad():
        for name in ("Mixed_5b", "Mixed_5c", "Mixed_5d", "Mixed_6a", "Mixed_6b", "Mixed_6c", "Mixed_6d", "Mixed_6e",
                     "Mixed_7a", "Mixed_7b", "Mixed_7c"):
            x = getattr(model, name)(x)
            widths.append(x.shape[1])
    assert widths == [256, 288, 288, 768, 768, 768, 768, 768, 1280, 2048, 2048] and x.shape[2:] == (8, 8)
    from torpor_amd.functions import inception as pinc
    om.load_numpy_state(om.InceptionV3(), pinc.init_weights())


def test_vgg16_counts_and_flattening():
    """138,357,544 parameters and 15.47 G multiply-accumulates per 224x224 image (published for
    configuration D); 13 convolutions of 3x3 with bias, 5 poolings, and fully connected layers on the
    channel-major flattening of the 512 x 7 x 7 map; the product-side weight generator loads strictly."""
    model = om.VGG16().eval()
    assert sum(p.numel() for p in model.parameters()) == 138357544
    m, y = _macs(model, torch.zeros(1, 3, 224, 224))
    assert y.shape == (1, 1000) and round(m / 1e9, 2) == 15.47
    convs = [c for c in model.modules() if isinstance(c, torch.nn.Conv2d)]
    assert len(convs) == 13 and all(c.kernel_size == (3, 3) and c.bias is not None for c in convs)
    assert sum(1 for c in model.modules() if isinstance(c, torch.nn.MaxPool2d)) == 5
    # flattening: feature (c, h, w) feeds classifier input c * 49 + h * 7 + w
    with torch.no_grad():
        for p in model.parameters():
            p.zero_()
        model.classifier[0].weight[5, 3 * 49 + 2 * 7 + 4] = 1.0
        f = torch.zeros(1, 512, 7, 7)
        f[0, 3, 2, 4] = 2.5
        h = model.classifier[0](torch.flatten(f, 1))
    assert h[0, 5] == 2.5 and h.abs().sum() == 2.5
    from torpor_amd.functions import vgg as pvgg
    om.load_numpy_state(om.VGG16(), pvgg.init_weights())


def test_squeezenet11_counts_and_fire_module():
    """1,235,496 parameters and 0.35 G multiply-accumulates per 224x224 image (published for revision 1.1),
    eight fire modules; a fire module is relu(squeeze) followed by relu(1x1) and relu(3x3) side by side."""
    model = om.SqueezeNet11().eval()
    assert sum(p.numel() for p in model.parameters()) == 1235496
    m, y = _macs(model, torch.zeros(1, 3, 224, 224))
    assert y.shape == (1, 1000) and round(m / 1e9, 2) == 0.35
    fires = [f for f in model.modules() if isinstance(f, om._Fire)]
    assert len(fires) == 8
    assert [f.squeeze.out_channels for f in fires] == [16, 16, 32, 32, 48, 48, 64, 64]
    torch.manual_seed(2)
    f = om._Fire(12, 4, 6, 10).eval()
    x = torch.randn(2, 12, 7, 5)
    with torch.no_grad():
        s_ = F.relu(F.conv2d(x, f.squeeze.weight, f.squeeze.bias))
        want = torch.cat([F.relu(F.conv2d(s_, f.expand1x1.weight, f.expand1x1.bias)),
                          F.relu(F.conv2d(s_, f.expand3x3.weight, f.expand3x3.bias, padding=1))], 1)
        assert torch.allclose(f(x), want, atol=1e-6)
    # map sizes at 224: 111 after the stem, 55 / 27 / 13 after the three ceil-mode poolings
    sizes, t = [], torch.zeros(1, 3, 224, 224)
    with torch.no_grad():
        for layer in model.features:
            t = layer(t)
            if isinstance(layer, (torch.nn.Conv2d, torch.nn.MaxPool2d)):
                sizes.append(t.shape[-1])
    assert sizes == [111, 55, 27, 13]
    from torpor_amd.functions import squeezenet as psq
    om.load_numpy_state(om.SqueezeNet11(), psq.init_weights())
