"""End to end over the reference's request flow on the GPU: a function container process talks
ZMTP/proto3 to a separate torpor_server process; results must equal the in-process C-ABI path
bit for bit and the PyTorch CPU oracle within rel 1e-3."""
import os
import signal
import subprocess
import tempfile

import numpy as np
import pytest
import torch

from oracle import models as om
from tests.harness import assert_close
from torpor_amd import client as wire
from torpor_amd.functions import bert, mobilenet, resnet
from torpor_amd.server import ACK_OK, Server

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SERVER_BIN = os.path.join(ROOT, "torpor_amd", "bin", "torpor_server")


@pytest.fixture(scope="module")
def gpu_wire_server():
    d = tempfile.mkdtemp(prefix="tpipc")
    env = dict(os.environ, TORPOR_IPC_DIR=d, TORPOR_MEM_LIMIT_BYTES=str(2 << 30), TORPOR_POOL_BYTES=str(3 << 30))
    p = subprocess.Popen([SERVER_BIN], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    line = p.stdout.readline()
    assert b"listening" in line, line
    yield d
    p.send_signal(signal.SIGTERM)
    try:
        p.wait(timeout=20)
    except subprocess.TimeoutExpired:
        p.kill()


def test_resnet50_over_the_wire(gpu_wire_server):
    weights = resnet.init_weights("resnet50", seed=5)
    x = torch.randn(1, 3, 96, 96, generator=torch.Generator().manual_seed(5)).numpy()
    with Server(mem_limit_bytes=1 << 30, pool_bytes=2 << 30) as local:
        (want_local,) = resnet.ResNet(local, 0, "resnet50", batch=1, weights=weights, image=96).register([x])
    with wire.RemoteServer(gpu_wire_server, client_id=7) as rs:
        fn = resnet.ResNet(rs, 7, "resnet50", batch=1, weights=weights, image=96)
        (first,) = fn.register([x])
        assert np.array_equal(first, want_local), "wire path differs from the in-process path"
        model = om.load_numpy_state(om.ResNet("resnet50"), weights)
        with torch.no_grad():
            want = model(torch.from_numpy(x)).numpy()
        assert_close(first, want, 1e-3, "resnet50 logits over the wire")
        (warm,) = fn.invoke([x], replay=False)            # op by op, batched messages
        assert np.array_equal(warm, first)
        assert fn.unload()[:2] == (ACK_OK, -1)
        (cold,) = fn.invoke([x])                          # swapped out -> one Replay message
        assert np.array_equal(cold, first)
        assert fn.unload()[0] == ACK_OK


def test_bert_small_over_the_wire(gpu_wire_server):
    cfg = dict(layers=2, hidden=128, heads=4, ffn=256)
    weights = bert.init_weights(seed=2, vocab=500, max_pos=64, cfg=cfg)
    ids = torch.randint(0, 500, (2, 48), generator=torch.Generator().manual_seed(1)).numpy()
    with wire.RemoteServer(gpu_wire_server, client_id=8) as rs:
        fn = bert.Bert(rs, 8, batch=2, seq=48, weights=weights, cfg=cfg)
        hidden, pooled = fn.register([ids])
        model = om.load_numpy_state(om.Bert(vocab=500, max_pos=64, **cfg), weights)
        with torch.no_grad():
            wh, wp = model(torch.from_numpy(ids))
        assert_close(hidden, wh.numpy(), 1e-3, "hidden")
        assert_close(pooled, wp.numpy(), 1e-3, "pooled")
        fn.unload()
        h2, p2 = fn.invoke([ids])
        assert np.array_equal(h2, hidden) and np.array_equal(p2, pooled)
        fn.unload()


def test_densenet_and_mobilenet_over_the_wire(gpu_wire_server):
    """The wire fields added for channel-slice views (conv x_pitch / y_pitch, batch-norm x_pitch,
    groups) and the op ids of window pooling / strided copy: results over the wire must equal the
    in-process C-ABI path bit for bit."""
    from torpor_amd.functions import densenet, mobilenet
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, 3, 64, 64, generator=g).numpy()
    for fid, make, weights in (
            (9, lambda s, f, w: densenet.DenseNet(s, f, "densenet121", batch=1, weights=w, image=64),
             densenet.init_weights("densenet121", seed=4)),
            (10, lambda s, f, w: mobilenet.MobileNetV2(s, f, batch=1, weights=w, image=64), mobilenet.init_weights(seed=4))):
        with Server(mem_limit_bytes=1 << 30, pool_bytes=2 << 30) as local:
            (want_local,) = make(local, 0, weights).register([x])
        with wire.RemoteServer(gpu_wire_server, client_id=fid) as rs:
            fn = make(rs, fid, weights)
            (first,) = fn.register([x])
            assert np.array_equal(first, want_local), "wire path differs from the in-process path"
            assert fn.unload()[0] == ACK_OK
            (cold,) = fn.invoke([x])
            assert np.array_equal(cold, first)
            assert fn.unload()[0] == ACK_OK


def test_router_over_the_wire(gpu_wire_server):
    """The router with one wire connection per function (the reference's function containers are
    separate clients of the server): FIFO trace, answers equal to the registration run."""
    from torpor_amd import router as R

    def factory(conn, fid, level):
        if fid % 2:
            return mobilenet.MobileNetV2(conn, fid, batch=1, seed=fid, level=level, image=64)
        return resnet.ResNet(conn, fid, "resnet50", batch=1, seed=fid, level=level, image=64)

    be = R.FunctionBackend(lambda fid: wire.RemoteServer(gpu_wire_server, client_id=fid), factory, R.ones_inputs)
    r = R.Router(be, slo_percentile=0.9, deadline_s=0.1, batch_limit=1, policy="fifo")
    try:
        for f in (20, 21, 22):
            r.launch(f, level=1)
        for f in (20, 21, 22):
            r.force_evict(f)
        arrivals = [(0.002, 20 + (i * 7) % 3) for i in range(90)]
        R.serve_arrivals(r, arrivals)
        out = r.summary()
        assert out["requests"] == 90 and out["queued"] == 0
        for f in (20, 21, 22):
            for a, b in zip(be.first[f], be.outputs(f)):
                assert np.array_equal(a, b), f"function {f} changed its answer over the wire"
            r.force_evict(f)
    finally:
        be.close()
