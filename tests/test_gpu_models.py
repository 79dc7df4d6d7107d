"""Whole-function parity on the GPU: logits against the plain PyTorch CPU forward of the same
seeded weights and inputs (rel 1e-3, fp32), swapped weights byte-identical to the host copy,
and warm / cold / replayed requests bit-identical to each other."""
import numpy as np
import pytest
import torch

from oracle import models as om
from tests.harness import assert_close
from torpor_amd.functions import bert, densenet, efficientnet, inception, mobilenet, resnet, squeezenet, vgg

pytestmark = pytest.mark.gpu
LOGIT_RTOL = 1e-3   # north-star bar: rel 1e-3 (fp32) on logits


def _perturb_bn(weights, seed):
    """Non-trivial batch-norm statistics, so that a wrong BN fold cannot pass."""
    rng = np.random.default_rng(seed)
    for k in list(weights):
        n = weights[k].shape
        if k.endswith("running_var"):
            weights[k] = rng.uniform(0.5, 1.5, n).astype(np.float32)
        elif k.endswith("running_mean"):
            weights[k] = (rng.standard_normal(n) * 0.1).astype(np.float32)
        elif len(n) == 1 and (k[:-len(".weight")] + ".running_var" in weights or k[:-len(".bias")] + ".running_var" in weights):
            if k.endswith(".weight"):
                weights[k] = rng.uniform(0.8, 1.2, n).astype(np.float32)
            elif k.endswith(".bias"):
                weights[k] = (rng.standard_normal(n) * 0.1).astype(np.float32)
    return weights


def _check_swap_identity(server, fn, weights):
    """Every uploaded tensor sits, byte for byte, at its image offset in the host store and in
    the device copy read back from HBM."""
    host = server.host_weights(fn.fid)
    dev = server.readback_weights(fn.fid)
    assert host.nbytes == dev.nbytes
    assert np.array_equal(host, dev), "device weight image differs from the host copy"
    for name, arr in weights.items():
        if name not in fn.w:
            continue
        raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
        off = server.weight_offset(fn.fid, fn.w[name])
        assert np.array_equal(dev[off:off + raw.size], raw), name


def _cycle(server, fn, inputs, first):
    """warm replay, warm op-by-op, cold replay: all bit-identical to the tracked first run."""
    warm = fn.invoke(inputs)
    for a, b in zip(first, warm):
        assert np.array_equal(a, b), "warm replay differs from the first run"
    warm2 = fn.invoke(inputs, replay=False)
    for a, b in zip(first, warm2):
        assert np.array_equal(a, b), "op-by-op request differs from the first run"
    ack, resp, _ = fn.unload()
    assert ack == 0 and resp == -1 and not server.resident(fn.fid)
    cold = fn.invoke(inputs)
    assert server.resident(fn.fid)
    for a, b in zip(first, cold):
        assert np.array_equal(a, b), "cold (swap-in) request differs from the first run"
    st = server.swap_stats(fn.fid)
    image = server.model_info(fn.fid)["image_bytes"]
    assert 0.8 * image < st["bytes"] <= image and st["copy_ms"] > 0   # link bytes: packed or as they are
    return st


@pytest.mark.parametrize("arch,batch", [("resnet50", 1), ("resnet152", 8)])
def test_resnet(gpu_server, arch, batch):
    fid = {"resnet50": 1, "resnet152": 3}[arch]
    weights = _perturb_bn(resnet.init_weights(arch, seed=0), seed=1)
    x = torch.randn(batch, 3, 224, 224, generator=torch.Generator().manual_seed(0)).numpy()
    fn = resnet.ResNet(gpu_server, fid, arch, batch=batch, weights=weights)
    (logits,) = fn.register([x])
    model = om.load_numpy_state(om.ResNet(arch), weights)
    with torch.no_grad():
        want = model(torch.from_numpy(x)).numpy()
    err = assert_close(logits, want, LOGIT_RTOL, f"{arch} logits")
    print(f"{arch} b{batch}: logits rel err {err:.2e}")
    info = gpu_server.model_info(fid)
    n_params = sum(int(np.prod(v.shape)) for k, v in weights.items() if "running" not in k)
    assert n_params == {"resnet50": 25557032, "resnet152": 60192808}[arch]
    assert info["param_bytes"] == sum(v.nbytes for v in weights.values())
    _check_swap_identity(gpu_server, fn, weights)
    _cycle(gpu_server, fn, [x], [logits])
    _check_swap_identity(gpu_server, fn, weights)
    fn.unload()


@pytest.mark.parametrize("arch,batch,seq", [("bert-base", 1, 128), ("bert-large", 4, 384)])
def test_bert(gpu_server, arch, batch, seq):
    fid = {"bert-base": 2, "bert-large": 4}[arch]
    weights = bert.init_weights(arch, seed=0)
    ids = torch.randint(0, 30522, (batch, seq), generator=torch.Generator().manual_seed(0)).numpy()
    fn = bert.Bert(gpu_server, fid, arch, batch=batch, seq=seq, weights=weights)
    hidden, pooled = fn.register([ids])
    model = om.load_numpy_state(om.Bert(**bert.CONFIGS[arch]), weights)
    with torch.no_grad():
        want_h, want_p = model(torch.from_numpy(ids))
    e1 = assert_close(hidden, want_h.numpy(), LOGIT_RTOL, f"{arch} last hidden state")
    e2 = assert_close(pooled, want_p.numpy(), LOGIT_RTOL, f"{arch} pooled output")
    print(f"{arch} b{batch} s{seq}: rel err hidden {e1:.2e} pooled {e2:.2e}")
    n_params = sum(int(np.prod(v.shape)) for v in weights.values())
    assert n_params == {"bert-base": 109482240, "bert-large": 335141888}[arch]
    uploaded = fn.weights()   # query / key / value stacked per layer, everything else as in `weights`
    assert sum(v.size for v in uploaded.values()) == n_params
    qkv = uploaded["encoder.layer.0.attention.self.qkv.weight"]
    hdim = bert.CONFIGS[arch]["hidden"]
    assert np.array_equal(qkv[hdim:2 * hdim], weights["encoder.layer.0.attention.self.key.weight"])
    _check_swap_identity(gpu_server, fn, uploaded)
    _cycle(gpu_server, fn, [ids], [hidden, pooled])
    _check_swap_identity(gpu_server, fn, uploaded)
    fn.unload()


@pytest.mark.parametrize("heads", [2, 4])
def test_bert_qa_with_token_types_and_mask(gpu_server, heads):
    """The question-answering head with token type ids and a padding mask (the call the
    reference's endpoint makes, tests/endpoint.py:52-57), head width 64 (fused attention) and
    32 (batched GEMMs + softmax), against the PyTorch oracle."""
    cfg = dict(layers=2, hidden=128, heads=heads, ffn=256)
    B, S = 3, 40
    weights = bert.init_weights(seed=5, vocab=300, max_pos=64, cfg=cfg, qa_head=True)
    g = torch.Generator().manual_seed(7)
    ids = torch.randint(0, 300, (B, S), generator=g).numpy()
    tt = torch.randint(0, 2, (B, S), generator=g).numpy()
    am = np.ones((B, S), np.int64)
    am[0, 29:] = 0
    am[2, 8:] = 0
    fn = bert.Bert(gpu_server, 11, batch=B, seq=S, weights=weights, cfg=cfg, token_types=True, masked=True)
    inputs = [ids, tt, bert.Bert.additive_mask(am)]
    start, end = fn.register(inputs)
    model = om.load_numpy_state(om.Bert(vocab=300, max_pos=64, qa_head=True, **cfg), weights)
    with torch.no_grad():
        want_s, want_e = model(torch.from_numpy(ids), torch.from_numpy(tt), torch.from_numpy(am))
    assert start.shape == (B, S)
    assert_close(start, want_s.numpy(), LOGIT_RTOL, "start logits")
    assert_close(end, want_e.numpy(), LOGIT_RTOL, "end logits")
    _cycle(gpu_server, fn, inputs, [start, end])
    fn.unload()


def test_resnet101(gpu_server):
    """ResNet-101 (served by the reference next to -50 and -152, tests/endpoint.py:16-29)."""
    weights = _perturb_bn(resnet.init_weights("resnet101", seed=2), seed=3)
    x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(4)).numpy()
    fn = resnet.ResNet(gpu_server, 12, "resnet101", batch=1, weights=weights)
    (logits,) = fn.register([x])
    model = om.load_numpy_state(om.ResNet("resnet101"), weights)
    with torch.no_grad():
        want = model(torch.from_numpy(x)).numpy()
    assert_close(logits, want, LOGIT_RTOL, "resnet101 logits")
    _cycle(gpu_server, fn, [x], [logits])
    fn.unload()


@pytest.mark.parametrize("arch,image,batch", [("densenet121", 64, 2), ("densenet169", 224, 1), ("densenet201", 224, 1)])
def test_densenet(gpu_server, arch, image, batch):
    """DenseNet (served by the reference, tests/endpoint.py:20-23): dense blocks built in place in one
    wide buffer (pitched batch-norm input, convolution output into a channel slice)."""
    weights = _perturb_bn(densenet.init_weights(arch, seed=6), seed=7)
    x = torch.randn(batch, 3, image, image, generator=torch.Generator().manual_seed(8)).numpy()
    fn = densenet.DenseNet(gpu_server, 13, arch, batch=batch, weights=weights, image=image)
    (logits,) = fn.register([x])
    model = om.load_numpy_state(om.DenseNet(arch), weights)
    with torch.no_grad():
        want = model(torch.from_numpy(x)).numpy()
    e = assert_close(logits, want, LOGIT_RTOL, f"{arch} logits")
    print(f"{arch} b{batch} {image}px: rel err {e:.2e}")
    _check_swap_identity(gpu_server, fn, weights)
    _cycle(gpu_server, fn, [x], [logits])
    fn.unload()


@pytest.mark.parametrize("family", ["densenet", "efficientnet"])
def test_fused_operand_transform_is_taken_and_agrees_with_the_separate_launches(gpu_server, family):
    """DenseNet's batch-norm + ReLU and EfficientNet's channel gate ride in the 1x1 convolution that follows
    them (TP_OP_BN_CONV1X1): fewer recorded ops than with `fused=False`, the same logits within the bar."""
    x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(21)).numpy()
    out, ops = {}, {}
    for fused in (False, None):
        if family == "densenet":
            weights = _perturb_bn(densenet.init_weights("densenet121", seed=6), seed=7)
            fn = densenet.DenseNet(gpu_server, 23, "densenet121", batch=1, weights=weights, fused=fused)
        else:
            weights = _perturb_bn(efficientnet.init_weights(seed=12), seed=13)
            fn = efficientnet.EfficientNetB0(gpu_server, 23, batch=1, weights=weights, fused=fused)
        (out[fused],) = fn.register([x])
        ops[fused] = gpu_server.model_info(23)["n_ops"]
        fn.unload()
    # DenseNet-121: 58 dense layers + 3 transitions lose a launch each; EfficientNet-B0: 11 of 16 blocks
    assert ops[None] <= ops[False] - (61 if family == "densenet" else 11), ops
    assert_close(out[None], out[False].astype(np.float64), LOGIT_RTOL, f"{family}: fused against separate launches")


@pytest.mark.parametrize("image,batch", [(96, 2), (224, 1)])
def test_mobilenet_v2(gpu_server, image, batch):
    """MobileNetV2 (tests/endpoint.py:30-31): depthwise convolutions, relu6, linear bottlenecks."""
    weights = _perturb_bn(mobilenet.init_weights(seed=9), seed=10)
    x = torch.randn(batch, 3, image, image, generator=torch.Generator().manual_seed(11)).numpy()
    fn = mobilenet.MobileNetV2(gpu_server, 14, batch=batch, weights=weights, image=image)
    (logits,) = fn.register([x])
    model = om.load_numpy_state(om.MobileNetV2(), weights)
    with torch.no_grad():
        want = model(torch.from_numpy(x)).numpy()
    e = assert_close(logits, want, LOGIT_RTOL, "mobilenet_v2 logits")
    print(f"mobilenet_v2 b{batch} {image}px: rel err {e:.2e}")
    _check_swap_identity(gpu_server, fn, weights)
    _cycle(gpu_server, fn, [x], [logits])
    fn.unload()


@pytest.mark.parametrize("image,batch", [(96, 2), (224, 1)])
def test_efficientnet_b0(gpu_server, image, batch):
    """EfficientNet-B0 (tests/endpoint.py:34-35): depthwise 3x3 / 5x5, SiLU, squeeze-and-excitation."""
    weights = _perturb_bn(efficientnet.init_weights(seed=12), seed=13)
    x = torch.randn(batch, 3, image, image, generator=torch.Generator().manual_seed(14)).numpy()
    fn = efficientnet.EfficientNetB0(gpu_server, 15, batch=batch, weights=weights, image=image)
    (logits,) = fn.register([x])
    model = om.load_numpy_state(om.EfficientNetB0(), weights)
    with torch.no_grad():
        want = model(torch.from_numpy(x)).numpy()
    e = assert_close(logits, want, LOGIT_RTOL, "efficientnet_b0 logits")
    print(f"efficientnet_b0 b{batch} {image}px: rel err {e:.2e}")
    _check_swap_identity(gpu_server, fn, weights)
    _cycle(gpu_server, fn, [x], [logits])
    fn.unload()


@pytest.mark.parametrize("image,batch", [(139, 2), (299, 1)])
def test_inception_v3(gpu_server, image, batch):
    """Inception-v3 (tests/endpoint.py:32-33): asymmetric convolutions, window pooling, branches
    written straight into channel slices of the block output."""
    weights = _perturb_bn(inception.init_weights(seed=15), seed=16)
    x = torch.randn(batch, 3, image, image, generator=torch.Generator().manual_seed(17)).numpy()
    fn = inception.InceptionV3(gpu_server, 16, batch=batch, weights=weights, image=image)
    (logits,) = fn.register([x])
    model = om.load_numpy_state(om.InceptionV3(), weights)
    with torch.no_grad():
        want = model(torch.from_numpy(x)).numpy()
    e = assert_close(logits, want, LOGIT_RTOL, "inception_v3 logits")
    print(f"inception_v3 b{batch} {image}px: rel err {e:.2e}")
    _check_swap_identity(gpu_server, fn, weights)
    _cycle(gpu_server, fn, [x], [logits])
    fn.unload()


def test_bert_large_question_answering_at_the_endpoints_size(gpu_server):
    """The reference endpoint's own BERT call at full size (tests/endpoint.py:36-40,52-57): BERT-large with
    the span head, batch 1, 512 tokens, token type ids."""
    arch, B, S = "bert-large", 1, 512
    weights = bert.init_weights(arch, seed=3, qa_head=True)
    g = torch.Generator().manual_seed(21)
    ids = torch.randint(0, 30522, (B, S), generator=g).numpy()
    tt = torch.randint(0, 2, (B, S), generator=g).numpy()
    fn = bert.Bert(gpu_server, 17, arch, batch=B, seq=S, weights=weights, token_types=True)
    start, end = fn.register([ids, tt])
    model = om.load_numpy_state(om.Bert(qa_head=True, **bert.CONFIGS[arch]), weights)
    with torch.no_grad():
        want_s, want_e = model(torch.from_numpy(ids), torch.from_numpy(tt))
    assert start.shape == (B, S) and end.shape == (B, S)
    e1 = assert_close(start, want_s.numpy(), LOGIT_RTOL, "span start logits")
    e2 = assert_close(end, want_e.numpy(), LOGIT_RTOL, "span end logits")
    print(f"bert-large QA b{B} s{S}: rel err start {e1:.2e} end {e2:.2e}")
    _check_swap_identity(gpu_server, fn, fn.weights())
    _cycle(gpu_server, fn, [ids, tt], [start, end])
    fn.unload()


def test_vgg16(gpu_server):
    """VGG-16 (tests/endpoint.py:26-27): 3x3 convolutions with bias, 2x2 max-pooling, 411 MB first fully
    connected layer on the channel-major flattening."""
    weights = vgg.init_weights(seed=18)
    rng = np.random.default_rng(19)
    for k in weights:   # non-zero biases, so that a dropped bias cannot pass
        if k.endswith(".bias"):
            weights[k] = (rng.standard_normal(weights[k].shape) * 0.05).astype(np.float32)
    x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(20)).numpy()
    fn = vgg.VGG16(gpu_server, 18, batch=1, weights=weights)
    (logits,) = fn.register([x])
    model = om.load_numpy_state(om.VGG16(), weights)
    with torch.no_grad():
        want = model(torch.from_numpy(x)).numpy()
    e = assert_close(logits, want, LOGIT_RTOL, "vgg16 logits")
    print(f"vgg16 b1: rel err {e:.2e}")
    assert gpu_server.model_info(18)["param_bytes"] == 4 * 138357544
    _check_swap_identity(gpu_server, fn, weights)
    _cycle(gpu_server, fn, [x], [logits])
    fn.unload()


@pytest.mark.parametrize("image,batch", [(96, 2), (224, 1)])
def test_squeezenet11(gpu_server, image, batch):
    """SqueezeNet 1.1 (tests/endpoint.py:20-21): fire modules whose two expansions write into the halves
    of one buffer."""
    weights = squeezenet.init_weights(seed=22)
    rng = np.random.default_rng(23)
    for k in weights:
        if k.endswith(".bias"):
            weights[k] = (rng.standard_normal(weights[k].shape) * 0.05).astype(np.float32)
    weights["classifier.1.weight"] = (weights["classifier.1.weight"] * 5).astype(np.float32)   # logits of a visible size
    x = torch.randn(batch, 3, image, image, generator=torch.Generator().manual_seed(24)).numpy()
    fn = squeezenet.SqueezeNet11(gpu_server, 19, batch=batch, weights=weights, image=image)
    (logits,) = fn.register([x])
    model = om.load_numpy_state(om.SqueezeNet11(), weights)
    with torch.no_grad():
        want = model(torch.from_numpy(x)).numpy()
    e = assert_close(logits, want, LOGIT_RTOL, "squeezenet1_1 logits")
    print(f"squeezenet1_1 b{batch} {image}px: rel err {e:.2e}")
    _check_swap_identity(gpu_server, fn, weights)
    _cycle(gpu_server, fn, [x], [logits])
    fn.unload()


def test_image_is_in_first_access_order(gpu_server):
    """ResNet uploads `downsample` after `conv3` (state-dict order) but uses it before: after
    registration the image must hold the tensors in the order the tracked run touched them."""
    weights = resnet.init_weights("resnet50", seed=3)
    x = np.zeros((1, 3, 64, 64), np.float32)
    fn = resnet.ResNet(gpu_server, 9, "resnet50", batch=1, weights=weights, image=64)
    fn.register([x])
    off = {k: gpu_server.weight_offset(9, va) for k, va in fn.w.items()}
    assert off["conv1.weight"] == 0
    assert off["layer1.0.downsample.0.weight"] < off["layer1.0.conv3.weight"]
    assert off["layer1.0.conv2.weight"] < off["layer1.0.downsample.0.weight"]
    assert off["fc.bias"] == max(off.values())
    ordered = sorted(off.values())
    sizes = {off[k]: weights[k].nbytes for k in off}
    for a, b in zip(ordered, ordered[1:]):
        assert a % 256 == 0 and a + sizes[a] <= b
    fn.unload()
