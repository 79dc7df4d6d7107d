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


@pytest.mark.parametrize("policy", ["sa", "fifo"])
def test_router_serves_a_fleet_under_memory_pressure(policy):
    with Server(mem_limit_bytes=260 << 20, pool_bytes=512 << 20) as s:
        be = R.FunctionBackend(s, _factory, R.ones_inputs)
        r = R.Router(be, slo_percentile=0.9, deadline_s=0.05, batch_limit=2, policy=policy)
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
        st1 = s.pool_stats()
        assert st1["swap_ins"] - st0["swap_ins"] >= 6 and st1["evictions"] > st0["evictions"]   # 3 ResNets exceed the budget
        for f in range(6):
            for a, b in zip(be.first[f], be.outputs(f)):      # the last request served during the trace
                assert np.array_equal(a, b), f"function {f} changed its answer"
            be.execute(f, 1)
            for a, b in zip(be.first[f], be.outputs(f)):
                assert np.array_equal(a, b), f"function {f} changed its answer"
        assert sum(k * v for k, v in out["batches"].items()) == 600
