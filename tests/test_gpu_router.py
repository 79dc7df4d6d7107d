"""The router in front of a real server on the GPU: a mixed fleet under a budget that forces swaps,
light functions (level 0) evicted before median ones, answers unchanged by queueing and swapping."""
import numpy as np
import pytest

from torpor_amd import router as R
from torpor_amd.functions import mobilenet, resnet
from torpor_amd.server import Server

pytestmark = pytest.mark.gpu


def _factory(server, fid, level):
    if fid % 2:
        return mobilenet.MobileNetV2(server, fid, batch=2, seed=fid, level=level, image=64)
    return resnet.ResNet(server, fid, "resnet50", batch=2, seed=fid, level=level, image=64)


def _same_rows(first, got, f):
    """Full batches replay the recorded stream (same bits); a smaller batch runs other tile shapes,
    so its rows agree with the registered run to rounding (inputs are all ones: every row is alike)."""
    if got.shape == first.shape:
        assert np.array_equal(first, got), f"function {f} changed its answer"
    else:
        ref = first[:got.shape[0]]
        assert np.abs(got - ref).max() <= 1e-4 * max(np.abs(ref).max(), 1e-6), f"function {f}: rows differ"


def test_fewer_rows_than_the_registered_batch():
    """`invoke_rows` runs a request at its own batch size inside the buffers of the registered one:
    same bits as a function registered at that size, and the oracle's answer."""
    import torch
    from oracle import models as om
    from tests.harness import assert_close
    w = resnet.init_weights("resnet50", seed=11)
    x = np.random.default_rng(11).standard_normal((4, 3, 64, 64)).astype(np.float32)
    model = om.load_numpy_state(om.ResNet("resnet50"), w)
    with torch.no_grad():
        want = model(torch.from_numpy(x)).numpy()
    with Server(mem_limit_bytes=1 << 30, pool_bytes=2 << 30) as s:
        big = resnet.ResNet(s, 0, "resnet50", batch=4, weights=w, image=64)
        (y4,) = big.register([x])
        assert_close(y4, want, 1e-3, "batch 4")
        for rows in (1, 2, 3):
            small = resnet.ResNet(s, rows, "resnet50", batch=rows, weights=w, image=64)
            (ys,) = small.register([x[:rows]])
            (got,) = big.invoke_rows([x[:rows]], rows)
            assert got.shape == (rows, 1000) and np.array_equal(got, ys), rows
            assert_close(got, want[:rows], 1e-3, f"{rows} rows")
        (again,) = big.invoke([x])                         # the recorded stream is untouched
        assert np.array_equal(again, y4)
        (cold,) = (big.unload(), big.invoke_rows([x[1:3]], 2))[1]   # also from the swapped-out state
        assert_close(cold, want[1:3], 1e-3, "rows 1..2 cold")
        with pytest.raises(ValueError):
            big.invoke_rows([x], 5)


def test_fewer_rows_bert_and_mobilenet():
    """The same for a transformer (rows = sequences) and a depthwise network."""
    from torpor_amd.functions import bert
    cfg = dict(layers=2, hidden=128, heads=2, ffn=256)
    wb = bert.init_weights(seed=3, vocab=400, max_pos=64, cfg=cfg)
    ids = np.random.default_rng(3).integers(0, 400, (4, 48))
    wm = mobilenet.init_weights(seed=6)
    xm = np.random.default_rng(6).standard_normal((3, 3, 64, 64)).astype(np.float32)
    with Server(mem_limit_bytes=1 << 30, pool_bytes=2 << 30) as s:
        big = bert.Bert(s, 0, batch=4, seq=48, weights=wb, cfg=cfg)
        big.register([ids])
        for rows in (1, 3):
            small = bert.Bert(s, 10 + rows, batch=rows, seq=48, weights=wb, cfg=cfg)
            want = small.register([ids[:rows]])
            got = big.invoke_rows([ids[:rows]], rows)
            assert all(np.array_equal(a, b) for a, b in zip(got, want)), rows
        mb = mobilenet.MobileNetV2(s, 1, batch=3, weights=wm, image=64)
        mb.register([xm])
        small = mobilenet.MobileNetV2(s, 21, batch=2, weights=wm, image=64)
        (want,) = small.register([xm[:2]])
        (got,) = mb.invoke_rows([xm[:2]], 2)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("miss_aware", [False, True])
@pytest.mark.parametrize("policy", ["sa", "fifo"])
def test_router_serves_a_fleet_under_memory_pressure(policy, miss_aware):
    """(miss_aware: requests of resident models are served while a swapped-out one streams in; same answers.)"""
    with Server(mem_limit_bytes=260 << 20, pool_bytes=512 << 20) as s:
        be = R.FunctionBackend(s, _factory, R.ones_inputs)
        r = R.Router(be, slo_percentile=0.9, deadline_s=0.05, batch_limit=2, policy=policy, miss_aware=miss_aware)
        for f in range(6):
            r.launch(f, level=0 if f % 2 else 1)
        for f in range(6):
            r.force_evict(f)
        assert not any(s.resident(f) for f in range(6))
        rng = np.random.default_rng(0)
        arrivals = [(g / 40, f) for g, f in R.fixed_rate_arrivals(6, 100, 1, rng)]   # 600 requests in 1.5 s
        st0 = s.pool_stats()
        wall = R.serve_arrivals(r, arrivals)
        out = r.summary()
        assert out["requests"] == 600 and out["queued"] == 0 and wall < 60
        assert out["dispatch"] == ("miss-aware" if miss_aware else "queue order") and (out["early_loads"] > 0) == miss_aware
        st1 = s.pool_stats()
        assert st1["swap_ins"] - st0["swap_ins"] >= 6 and st1["evictions"] > st0["evictions"]   # 3 ResNets exceed the budget
        assert set(out["batches"]) <= {1, 2}
        for f in range(6):
            for a, b in zip(be.first[f], be.outputs(f)):      # the last request served during the trace
                _same_rows(a, b, f)
            be.execute(f, 2)                                  # full batch: the recorded op stream, same bits
            for a, b in zip(be.first[f], be.outputs(f)):
                assert np.array_equal(a, b), f"function {f} changed its answer"
            be.execute(f, 1)                                  # one request: issued op by op at batch 1
            for a, b in zip(be.first[f], be.outputs(f)):
                assert b.shape[0] == 1
                _same_rows(a, b, f)
        assert sum(k * v for k, v in out["batches"].items()) == 600
