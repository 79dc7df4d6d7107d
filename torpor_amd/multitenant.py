"""Multi-tenant serving of one GPU: a fleet of registered functions, a seeded request trace, and the loop
that serves it.  The arrival process is that of the reference's load generator
(scripts/sender_fix_rate.py:46-56): exponential gaps at a fixed mean rate, here with Zipf popularity over
the functions.  Used by bench.py, bench_multitenant.py and the GPU tests of the 64-model configuration."""
import sys
import time

import numpy as np

# 32 ResNet-50 + 16 BERT-base (sequence 128) + 16 ResNet-152, seeds 0..63, batch 1
FLEET_64 = (32, 16, 16)


def fleet_plan(n_r50, n_bert, n_r152):
    return [("resnet50", "resnet")] * n_r50 + [("bert-base", "bert")] * n_bert + [("resnet152", "resnet")] * n_r152


def function_inputs(fid, family):
    """The seeded request of function `fid` (the same one a CPU re-computation of its answer uses)."""
    import torch
    g = torch.Generator().manual_seed(1000 + fid)
    if family == "resnet":
        return [torch.randn(1, 3, 224, 224, generator=g).numpy()]
    return [torch.randint(0, 30522, (1, 128), generator=g).numpy()]


def build_fleet(server, n_r50=32, n_bert=16, n_r152=16, levels=None, keep_weights=()):
    """Registers the functions (ids 0..n-1, weights seeded by the id); `levels` maps family name ->
    model level of the ExecuteAfterLoad payload (0 light, 1 median, 2 heavy; default: the functions'
    own default).  `keep_weights`: ids whose host-side weight dictionaries are kept for re-computation."""
    from torpor_amd.functions import bert, resnet

    fleet = []
    for fid, (arch, family) in enumerate(fleet_plan(n_r50, n_bert, n_r152)):
        kw = {}
        if levels is not None and arch in levels:
            kw["level"] = levels[arch]
        if family == "resnet":
            fn = resnet.ResNet(server, fid, arch, batch=1, seed=fid, **kw)
        else:
            fn = bert.Bert(server, fid, arch, batch=1, seq=128, seed=fid, **kw)
        inputs = function_inputs(fid, family)
        weights = fn._weights if fid in keep_weights else None   # as init_weights made them (the oracle twins load these)
        first = fn.register(inputs)
        fn._weights = None          # the server holds the authoritative copy now
        packed, outbuf, views = fn.pack(inputs, pinned=True)   # inputs and results in pinned memory, as a serving loop keeps them
        fleet.append(dict(fn=fn, fid=fid, arch=arch, family=family, inputs=inputs, weights=weights, packed=packed,
                          outbuf=outbuf, views=views, first=[a.copy() for a in first]))
    return fleet


def zipf_probs(n, s=1.1):
    p = 1.0 / np.arange(1, n + 1) ** s
    return p / p.sum()


def make_trace(n_functions, n_requests, rate, seed=0, zipf_s=1.1):
    """(arrival times in seconds, function id per request).  Popularity rank -> function id is a fixed
    shuffle, so that the hot functions are a mix of the model families."""
    rng = np.random.default_rng(seed)
    arrivals = np.cumsum(rng.exponential(1.0 / rate, n_requests))
    order = rng.permutation(n_functions)
    picks = order[rng.choice(n_functions, size=n_requests, p=zipf_probs(n_functions, zipf_s))]
    return arrivals, picks


def pct(xs, q):
    if not len(xs):
        return None
    xs = np.sort(np.asarray(xs))
    return float(xs[min(len(xs) - 1, int(round(q * (len(xs) - 1))))])


def serve(server, fleet, arrivals, picks, open_loop=True, check_every=500, after_request=None, note_every_s=30.0,
          lookahead=0, dispatch="in-order"):
    """dispatch="miss-aware": the open-loop trace through torpor_amd.dispatch.MissAwareDispatcher (requests of
    resident models are served while the swap-in of the oldest swapped-out one streams; see serve_miss_aware).
    Otherwise: serves the trace in arrival order on the single executor.  open_loop: a request is not issued before
    its arrival time and latency = completion - arrival (queueing included); otherwise requests run back to
    back and latency is the service time.  Every `check_every`-th answer is compared bit for bit with the
    function's registration run.  after_request(i, fid, hit) is called after each request.

    lookahead > 0 (open loop only): once a request has been started, the models of up to that many requests
    that are already waiting behind it are asked for with a Load request (the reference's prefetch signal,
    include/server/controller.hpp:208-215), so that their swap-ins queue behind this request's copies and
    run while it computes.  A request whose model arrived that way counts as a hit."""
    import gc

    from .server import REQ_LOAD
    if dispatch == "miss-aware":
        if not open_loop:
            raise ValueError("miss-aware dispatch reorders a queue of arrived requests: open loop only")
        return serve_miss_aware(server, fleet, arrivals, picks, check_every, after_request, note_every_s)
    n_req = len(picks)
    gc.collect()
    gc.disable()   # a collection of the interpreter inside a request (tens of milliseconds) is not the path's
    try:
        return _serve_in_order(server, fleet, arrivals, picks, open_loop, check_every, after_request, note_every_s,
                               lookahead, REQ_LOAD, n_req)
    finally:
        gc.enable()


def _serve_in_order(server, fleet, arrivals, picks, open_loop, check_every, after_request, note_every_s, lookahead,
                    REQ_LOAD, n_req):
    st0 = server.pool_stats()
    lat_hit, lat_miss, by_arch = [], [], {}
    swaps = _SwapMeter(server)
    prefetches = 0
    t0 = time.perf_counter()
    next_note = note_every_s
    for i in range(n_req):
        now = time.perf_counter() - t0
        if now >= next_note:        # a line now and then, so that a long run is seen to be alive
            print(f"[{now:6.0f} s] {i} of {n_req} requests served", file=sys.stderr, flush=True)
            next_note += note_every_s
        if open_loop and now < arrivals[i]:
            while time.perf_counter() - t0 < arrivals[i]:
                pass
        f = fleet[picks[i]]
        fid = f["fid"]
        hit = server.resident(fid)
        t_req = time.perf_counter()
        ack, _, dfr = server.signal(1, fid, "")
        assert ack == 0 and not dfr
        if lookahead and open_loop:
            now = time.perf_counter() - t0
            for j in range(i + 1, min(i + 1 + lookahead, n_req)):
                if arrivals[j] > now:
                    break
                nxt = fleet[picks[j]]["fid"]
                if nxt != fid and not server.resident(nxt):
                    prefetches += server.signal(REQ_LOAD, nxt, "")[0] == 0
        server.replay(fid, f["packed"], f["outbuf"])
        done = time.perf_counter()
        lat = ((done - t0 - arrivals[i]) if open_loop else (done - t_req)) * 1e3
        (lat_hit if hit else lat_miss).append(lat)
        by_arch.setdefault((f["arch"], hit), []).append(lat)
        if not hit:
            swaps.started(fid)
        swaps.collect()
        if check_every and i % check_every == 0:
            out = f["fn"].postprocess(f["views"])
            for a, b in zip(f["first"], out):
                if not np.array_equal(a, b):
                    raise AssertionError(f"function {fid}: answer changed after swapping")
        if after_request is not None:
            after_request(i, fid, hit)
    wall = time.perf_counter() - t0
    swaps.collect(wait=True)
    st1 = server.pool_stats()
    return _summary(server, n_req, wall, st0, st1, lat_hit, lat_miss, by_arch, swaps.bytes, swaps.ms,
                    dispatch="in-order", lookahead=lookahead, prefetches=int(prefetches))


class _SwapMeter:
    """Bytes and copy time of the swap-ins of a run.  A swap-in's figures are read once it has landed completely
    (tp_get_swap_stats waits for the last transfer group otherwise, and tables that a request does not wait for
    land up to 2 ms after the request has answered): asking right after the request would hold up the next one."""

    def __init__(self, server):
        self.server, self.pending, self.bytes, self.ms = server, set(), 0, 0.0

    def started(self, fid):
        self.pending.add(fid)

    def collect(self, wait=False):
        for fid in list(self.pending):
            if wait or self.server.loaded(fid) or not self.server.resident(fid):
                if self.server.resident(fid):
                    st = self.server.swap_stats(fid)
                    self.bytes += st["bytes"]
                    self.ms += st["copy_ms"]
                self.pending.discard(fid)


def _summary(server, n_req, wall, st0, st1, lat_hit, lat_miss, by_arch, swap_bytes, swap_ms, **extra):
    all_lat = lat_hit + lat_miss
    return dict(
        requests=n_req, wall_s=wall, achieved_rps=n_req / wall, **extra,
        hit_ratio=len(lat_hit) / max(n_req, 1), evictions=st1["evictions"] - st0["evictions"],
        fragmentation_evictions=st1["fragmentation_evictions"] - st0["fragmentation_evictions"],
        swap_ins=st1["swap_ins"] - st0["swap_ins"],
        latency_ms=dict(p50=pct(all_lat, 0.5), p99=pct(all_lat, 0.99), mean=float(np.mean(all_lat)) if all_lat else None),
        hit_ms=dict(p50=pct(lat_hit, 0.5), p99=pct(lat_hit, 0.99), n=len(lat_hit)),
        miss_ms=dict(p50=pct(lat_miss, 0.5), p99=pct(lat_miss, 0.99), n=len(lat_miss)),
        per_model_ms={f"{a}/{'hit' if h else 'miss'}": dict(p50=pct(v, 0.5), p99=pct(v, 0.99), n=len(v))
                      for (a, h), v in sorted(by_arch.items())},
        swap_gbps=(swap_bytes / 1e9) / (swap_ms * 1e-3) if swap_ms else None,
        pool_used_gib=st1["used"] / 2 ** 30, lru_models=st1["lru_models"],
        pinned_host_gib=(st1["host_image_bytes"] + st1["host_transfer_bytes"] + st1["host_staging_bytes"]) / 2 ** 30,
        device_outside_pool_gib=(st1["device_staging_bytes"] + st1["device_workspace_bytes"]) / 2 ** 30,
    )


def serve_miss_aware(server, fleet, arrivals, picks, check_every=500, after_request=None, note_every_s=30.0,
                     margin_s=0.0003):
    """The open-loop trace on the single executor, the queue of arrived requests ordered by
    torpor_amd.dispatch.MissAwareDispatcher: the oldest request of a swapped-out model gets its swap-in started
    with a Load signal (include/server/controller.hpp:208-215), requests of resident models run while it streams,
    and the waiting request is started when the rest of its copy is as long as its forward pass (both figures
    are the engine's: tp_get_load_estimate).  One function is active at a time, as in the reference.  A request
    counts as a miss when the swap-in was started for it; latency = completion - arrival."""
    import gc

    from .dispatch import MissAwareDispatcher
    from .server import REQ_LOAD
    n_req = len(picks)
    d = MissAwareDispatcher(margin_s=margin_s)
    est = {}
    st0 = server.pool_stats()
    lat_hit, lat_miss, by_arch = [], [], {}
    swaps = _SwapMeter(server)
    nxt = served = 0
    next_note = note_every_s
    resident = server.resident
    gc.collect()
    gc.disable()   # a collection of the interpreter inside a request (tens of milliseconds) is not the path's
    t0 = time.perf_counter()
    try:
        while served < n_req:
            now = time.perf_counter() - t0
            if now >= next_note:
                print(f"[{now:6.0f} s] {served} of {n_req} requests served", file=sys.stderr, flush=True)
                next_note += note_every_s
            while nxt < n_req and arrivals[nxt] <= now:
                d.arrive(nxt, fleet[picks[nxt]]["fid"], arrivals[nxt])
                nxt += 1
            kind, what = d.decide(now, resident)
            if kind == "load":
                fid = what.fid
                if fid not in est:
                    a, b = server.load_estimate(fid)
                    est[fid] = (a * 1e-3, b * 1e-3)
                if server.signal(REQ_LOAD, fid, "")[0] == 0:
                    d.load_started(fid, time.perf_counter() - t0, *est[fid])
                else:       # refused (nothing evictable): the request will bring its model in itself
                    d.load_started(fid, now, 0.0, 0.0)
                continue
            if kind == "idle":
                wake = arrivals[nxt] if nxt < n_req else None
                if what is not None and (wake is None or what < wake):
                    wake = what
                while time.perf_counter() - t0 < wake:
                    pass
                continue
            f = fleet[picks[what.seq]]
            fid = f["fid"]
            ack, _, dfr = server.signal(1, fid, "")
            assert ack == 0 and not dfr
            server.replay(fid, f["packed"], f["outbuf"])
            done = time.perf_counter() - t0
            lat = (done - what.arrival) * 1e3
            hit = not what.miss
            (lat_hit if hit else lat_miss).append(lat)
            by_arch.setdefault((f["arch"], hit), []).append(lat)
            if not hit:
                swaps.started(fid)
            swaps.collect()
            if check_every and what.seq % check_every == 0:
                out = f["fn"].postprocess(f["views"])
                for a, b in zip(f["first"], out):
                    if not np.array_equal(a, b):
                        raise AssertionError(f"function {fid}: answer changed after swapping")
            if after_request is not None:
                after_request(what.seq, fid, hit)
            served += 1
    finally:
        gc.enable()
    wall = time.perf_counter() - t0
    swaps.collect(wait=True)
    st1 = server.pool_stats()
    return _summary(server, n_req, wall, st0, st1, lat_hit, lat_miss, by_arch, swaps.bytes, swaps.ms,
                    dispatch="miss-aware", lookahead=0, prefetches=d.loads)


def run_cap(cap_gib, seconds, rate, models=FLEET_64, seed=0, pool_headroom_gib=2.0, lookahead=0, dispatch="in-order",
            **server_kw):
    """One engine with an LRU budget of `cap_gib`, the fleet registered, the open-loop trace served."""
    from torpor_amd.server import Server

    limit = int(cap_gib * 2 ** 30)
    with Server(mem_limit_bytes=limit, pool_bytes=limit + int(pool_headroom_gib * 2 ** 30), **server_kw) as server:
        link = server.measure_h2d(256 << 20, 5)
        t0 = time.perf_counter()
        fleet = build_fleet(server, *models)
        reg_s = time.perf_counter() - t0
        charged = sum(server.model_info(f["fid"])["total_bytes"] for f in fleet)
        weights = sum(server.model_info(f["fid"])["image_bytes"] for f in fleet)
        arrivals, picks = make_trace(len(fleet), int(seconds * rate), rate, seed)
        r = serve(server, fleet, arrivals, picks, lookahead=lookahead, dispatch=dispatch)
        r.update(cap_gib=cap_gib, cap_binds=charged >= limit, registration_s=reg_s, offered_rps=rate,
                 charged_total_gib=charged / 2 ** 30, weights_total_gb=weights / 1e9, link_peak_gbps=link)
        del fleet
    return r
