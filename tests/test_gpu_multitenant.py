"""The 64-model multi-tenant configuration on the device: 32 ResNet-50 + 16 BERT-base (sequence 128) +
16 ResNet-152, seeds 0..63, batch 1, a seeded Poisson (200 req/s) / Zipf(1.1) trace
(scripts/sender_fix_rate.py:46-56 is the arrival shape), under the configuration's own 24 GiB cap and
under a cap that binds (8 GiB), with the two-class eviction policy over model levels 0 / 1 / 2 and with
plain LRU (include/server/evictor.hpp:28-264, controller.hpp:103-109,141-152).

Checked: after every request the set of resident functions equals that of the oracle evictor
(oracle/host_ref.py) fed the same trace; sampled answers of every family equal the PyTorch CPU forward of
oracle/models.py (not just the registration run); every resident model's weights read back byte for byte."""
import numpy as np
import pytest

from oracle import models as om
from oracle.host_ref import IaRef, LruRef
from torpor_amd import multitenant as mt
from torpor_amd.functions import bert
from torpor_amd.server import Server

pytestmark = pytest.mark.gpu

N_REQ = 1000
RATE = 200.0
LEVELS = {"resnet50": 0, "bert-base": 1, "resnet152": 2}   # light / median / heavy


def _cpu_answer(f):
    import torch
    if f["family"] == "resnet":
        model = om.load_numpy_state(om.ResNet(f["arch"]), f["weights"])
        with torch.no_grad():
            return [model(torch.from_numpy(f["inputs"][0])).numpy()]
    model = om.load_numpy_state(om.Bert(**bert.CONFIGS[f["arch"]]), f["weights"])
    with torch.no_grad():
        return [o.numpy() for o in model(torch.from_numpy(f["inputs"][0]))]


def _rel_err(got, want):
    return float(np.abs(np.asarray(got, np.float64) - want).max() / max(float(np.abs(want).max()), 1e-30))


def _run(cap_gib, two_class):
    limit = int(cap_gib * 2 ** 30)
    sampled = (0, 17, 32, 40, 48, 63)        # two functions of each family, re-computed on the CPU
    # pool = twice the budget: the contiguous-extent fallback (victims beyond the policy's) must not occur
    with Server(mem_limit_bytes=limit, pool_bytes=2 * limit, evict_lru=not two_class) as s:
        fleet = mt.build_fleet(s, *mt.FLEET_64, levels=LEVELS, keep_weights=sampled)
        sizes = {f["fid"]: s.model_info(f["fid"])["total_bytes"] for f in fleet}
        ref = IaRef(1, limit) if two_class else LruRef(limit)

        def ref_add(fid):
            if two_class:
                ref.level[fid] = LEVELS[fleet[fid]["arch"]]
                return ref.check_and_add(0, fid, sizes[fid])
            return ref.check_and_add(fid, sizes[fid])

        def ref_set():
            if two_class:
                return {f for f, g in ref.gpus.items() if 0 in g}
            return set(ref.items)

        for f in fleet:                       # registration order: the eviction check of each finished cold start
            ref_add(f["fid"])
        assert {f["fid"] for f in fleet if s.resident(f["fid"])} == ref_set(), "after registration"
        arrivals, picks = mt.make_trace(len(fleet), N_REQ, RATE, seed=0)
        # Request by request, so that the oracle can be stepped in between: it sees check_and_add at each
        # Execute signal (the request's lock is taken and dropped within the request, so it never shields
        # anything from a later one).
        hits = 0
        for i in range(N_REQ):
            fid = int(picks[i])
            f = fleet[fid]
            want_hit = fid in ref_set()
            assert s.resident(fid) == want_hit, (i, fid)
            hits += want_hit
            ref_add(fid)
            ack, _, dfr = s.signal(1, fid, "")
            assert ack == 0 and not dfr
            s.replay(fid, f["packed"], f["outbuf"])
            got = {g["fid"] for g in fleet if s.resident(g["fid"])}
            assert got == ref_set(), (i, fid, sorted(got ^ ref_set()))
            if i % 97 == 0 or fid in sampled:
                out = f["fn"].postprocess(f["views"])
                for a, b in zip(f["first"], out):
                    assert np.array_equal(a, b), f"request {i}: function {fid} answers differently after swapping"
        st = s.pool_stats()
        assert st["fragmentation_evictions"] == 0
        assert st["lru_used"] == (ref.cur[0] if two_class else ref.cur)
        # answers against the PyTorch CPU forward, one cold and one warm request per sampled function
        for fid in sampled:
            f = fleet[fid]
            want = _cpu_answer(f)
            for cold in (True, False):
                if cold:
                    f["fn"].unload()
                    ref.force_evict(0, fid) if two_class else ref.force_evict(fid)
                ref_add(fid)
                got = f["fn"].invoke(f["inputs"])
                for a, b in zip(got, want):
                    assert _rel_err(a, b) <= 1e-3, (fid, f["arch"], cold, _rel_err(a, b))   # the stated bar, fp32
        assert {g["fid"] for g in fleet if s.resident(g["fid"])} == ref_set()
        # swapped weights are byte-identical to the host copy for everything resident at the end
        resident = [g["fid"] for g in fleet if s.resident(g["fid"])]
        assert len(resident) >= 8
        for fid in resident:
            assert np.array_equal(s.readback_weights(fid), s.host_weights(fid)), fid
        charged = sum(sizes.values())
        return dict(hit_ratio=hits / N_REQ, evictions=st["evictions"], swap_ins=st["swap_ins"], charged=charged,
                    resident=len(resident))


def test_64_models_under_the_configurations_24_gib_cap():
    r = _run(24.0, two_class=True)
    # what the cap charges (weights + activation arenas, whole 2 MiB slabs) is below 24 GiB: nothing is evicted
    assert r["charged"] < 24 * 2 ** 30 and r["evictions"] == 0 and r["hit_ratio"] == 1.0 and r["resident"] == 64


def test_64_models_under_a_binding_cap_two_class_policy_with_levels():
    r = _run(8.0, two_class=True)
    assert r["charged"] > 8 * 2 ** 30 and r["evictions"] > 50 and 0.3 < r["hit_ratio"] < 1.0


def test_64_models_under_a_binding_cap_plain_lru():
    r = _run(8.0, two_class=False)
    assert r["evictions"] > 50 and 0.3 < r["hit_ratio"] < 1.0


def test_prefetching_the_models_of_waiting_requests_changes_no_answer():
    """Load requests (controller.hpp:208-215) for the models of requests already waiting, issued while the current
    request runs: every answer still equals the function's registration run bit for bit, the budget holds after
    every request, and what is resident at the end reads back byte for byte."""
    limit = int(1.5 * 2 ** 30)
    with Server(mem_limit_bytes=limit, pool_bytes=2 * limit) as s:
        fleet = mt.build_fleet(s, 8, 4, 4)
        assert sum(s.model_info(f["fid"])["total_bytes"] for f in fleet) > 2 * limit      # the cap binds
        # arrivals faster than the executor serves them, so that requests do wait behind one another
        arrivals, picks = mt.make_trace(len(fleet), 600, 3000.0, seed=3)
        over = []

        def after(i, fid, hit):
            st = s.pool_stats()
            if st["lru_used"] > limit:
                over.append((i, st["lru_used"]))

        r0 = mt.serve(s, fleet, arrivals, picks, check_every=1, after_request=after, lookahead=0)
        r2 = mt.serve(s, fleet, arrivals, picks, check_every=1, after_request=after, lookahead=2)
        assert not over, over[:3]
        assert r0["prefetches"] == 0 and r2["prefetches"] > 20, (r0["prefetches"], r2["prefetches"])
        # a prefetched model counts as a hit; the margin allows for what a prefetch evicted that was asked for next
        assert r2["hit_ratio"] >= r0["hit_ratio"] - 0.05, (r0["hit_ratio"], r2["hit_ratio"])
        assert r2["fragmentation_evictions"] == 0
        resident = [f["fid"] for f in fleet if s.resident(f["fid"])]
        assert resident
        for fid in resident:
            assert np.array_equal(s.readback_weights(fid), s.host_weights(fid)), fid


def test_miss_aware_dispatch_changes_the_order_and_no_answer():
    """The same backlogged trace in arrival order and through the miss-aware dispatcher (hits served while the
    oldest miss's swap-in streams, Load signal of controller.hpp:208-215): every answer equals the function's
    registration run bit for bit either way, the budget holds after every request, requests of one function keep
    their order, what is resident at the end reads back byte for byte, and requests that found their model
    resident wait less in the tail."""
    limit = int(1.5 * 2 ** 30)
    with Server(mem_limit_bytes=limit, pool_bytes=2 * limit) as s:
        fleet = mt.build_fleet(s, 8, 4, 4)
        assert sum(s.model_info(f["fid"])["total_bytes"] for f in fleet) > 2 * limit      # the cap binds
        for f in fleet:                                   # the engine's own estimates, which the dispatcher plans with
            swap_ms, fwd_ms = s.load_estimate(f["fid"])
            assert 0.05 < swap_ms < 20 and 0.1 < fwd_ms < 20, (f["arch"], swap_ms, fwd_ms)
        arrivals, picks = mt.make_trace(len(fleet), 800, 500.0, seed=5)
        over, order = [], []

        def after(i, fid, hit):
            st = s.pool_stats()
            if st["lru_used"] > limit:
                over.append((i, st["lru_used"]))
            order.append((i, fid))

        r_io = mt.serve(s, fleet, arrivals, picks, check_every=1, after_request=after)
        order_io, order[:] = list(order), []
        r_ma = mt.serve(s, fleet, arrivals, picks, check_every=1, after_request=after, dispatch="miss-aware")
        assert not over, over[:3]
        assert [i for i, _ in order_io] == list(range(len(picks)))
        assert sorted(i for i, _ in order) == list(range(len(picks))) and [i for i, _ in order] != list(range(len(picks)))
        last = {}
        for i, fid in order:                              # per function: arrival order
            assert last.get(fid, -1) < i
            last[fid] = i
        assert r_ma["dispatch"] == "miss-aware" and r_ma["prefetches"] == r_ma["miss_ms"]["n"] > 20
        assert r_ma["hit_ms"]["p99"] < r_io["hit_ms"]["p99"], (r_ma["hit_ms"], r_io["hit_ms"])
        resident = [f["fid"] for f in fleet if s.resident(f["fid"])]
        assert resident
        for fid in resident:
            assert np.array_equal(s.readback_weights(fid), s.host_weights(fid)), fid
            assert s.loaded(fid)
