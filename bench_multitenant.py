#!/usr/bin/env python3
"""Multi-tenant serving benchmark on one MI355X (BASELINE.json configs[4]).

64 random-init models (32 ResNet-50, 16 BERT-base seq 128, 16 ResNet-152; seeds 0..63, batch 1)
are registered, so all weights sit in the pinned host store; requests then arrive as an open-loop
Poisson process (default 200 req/s) with Zipf(1.1) popularity over the 64 functions (the arrival
process of the reference's load generator, scripts/sender_fix_rate.py:46-56) and are served in
arrival order by the single executor.  Latency = completion - arrival, so it includes queueing.

What the pool cap charges: per resident model, its weight image plus its activation arena, each
rounded up to 2 MiB slabs (the reference also charges every block of a model,
include/server/model_repo.hpp:139-140).  The 64 models total about 14.6 GiB charged, so the
24 GiB cap of the config does not force evictions; the run is therefore repeated with a binding
cap (default 8 GiB) and both are reported.

Prints one JSON line.  Usage: python bench_multitenant.py [--seconds 60] [--rate 200] [--caps-gb 24 8]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def build_fleet(server, n_r50=32, n_bert=16, n_r152=16):
    import torch
    from torpor_amd.functions import bert, resnet

    fleet = []
    plan = [("resnet50", "resnet")] * n_r50 + [("bert-base", "bert")] * n_bert + [("resnet152", "resnet")] * n_r152
    for fid, (arch, family) in enumerate(plan):
        g = torch.Generator().manual_seed(1000 + fid)
        if family == "resnet":
            fn = resnet.ResNet(server, fid, arch, batch=1, seed=fid)
            inputs = [torch.randn(1, 3, 224, 224, generator=g).numpy()]
        else:
            fn = bert.Bert(server, fid, arch, batch=1, seq=128, seed=fid)
            inputs = [torch.randint(0, 30522, (1, 128), generator=g).numpy()]
        first = fn.register(inputs)
        fn._weights = None          # the server holds the authoritative copy now
        packed, outbuf, views = fn.pack(inputs)
        fleet.append(dict(fn=fn, arch=arch, packed=packed, outbuf=outbuf, views=views,
                          first=[a.copy() for a in first]))
    return fleet


def zipf_probs(n, s=1.1):
    p = 1.0 / np.arange(1, n + 1) ** s
    return p / p.sum()


def pct(xs, q):
    if not len(xs):
        return None
    xs = np.sort(np.asarray(xs))
    return float(xs[min(len(xs) - 1, int(round(q * (len(xs) - 1))))])


def serve(server, fleet, seconds, rate, seed, check_every=500):
    rng = np.random.default_rng(seed)
    n_req = int(seconds * rate)
    arrivals = np.cumsum(rng.exponential(1.0 / rate, n_req))
    # popularity rank -> function id: a fixed shuffle, so that hot functions are a mix of models
    order = rng.permutation(len(fleet))
    picks = order[rng.choice(len(fleet), size=n_req, p=zipf_probs(len(fleet)))]
    st0 = server.pool_stats()
    lat_hit, lat_miss, by_arch, swap_bytes, swap_ms = [], [], {}, 0, 0.0
    t0 = time.perf_counter()
    next_note = 30.0
    for i in range(n_req):
        now = time.perf_counter() - t0
        if now >= next_note:        # a line every half minute, so that a long run is seen to be alive
            print(f"[{now:6.0f} s] {i} of {n_req} requests served", file=sys.stderr, flush=True)
            next_note += 30.0
        if now < arrivals[i]:
            while time.perf_counter() - t0 < arrivals[i]:
                pass
        f = fleet[picks[i]]
        fid = f["fn"].fid
        hit = server.resident(fid)
        ack, _, dfr = server.signal(1, fid, "")
        assert ack == 0 and not dfr
        server.replay(fid, f["packed"], f["outbuf"])
        lat = (time.perf_counter() - t0 - arrivals[i]) * 1e3
        (lat_hit if hit else lat_miss).append(lat)
        by_arch.setdefault((f["arch"], hit), []).append(lat)
        if not hit:
            s = server.swap_stats(fid)
            swap_bytes += s["bytes"]
            swap_ms += s["copy_ms"]
        if i % check_every == 0:
            out = f["fn"].postprocess(f["views"])
            for a, b in zip(f["first"], out):
                if not np.array_equal(a, b):
                    raise SystemExit(f"function {fid}: answer changed after swapping")
    wall = time.perf_counter() - t0
    st1 = server.pool_stats()
    all_lat = lat_hit + lat_miss
    return dict(
        requests=n_req, wall_s=wall, achieved_rps=n_req / wall,
        hit_ratio=len(lat_hit) / n_req, evictions=st1["evictions"] - st0["evictions"],
        swap_ins=st1["swap_ins"] - st0["swap_ins"],
        latency_ms=dict(p50=pct(all_lat, 0.5), p99=pct(all_lat, 0.99), mean=float(np.mean(all_lat))),
        hit_ms=dict(p50=pct(lat_hit, 0.5), p99=pct(lat_hit, 0.99), n=len(lat_hit)),
        miss_ms=dict(p50=pct(lat_miss, 0.5), p99=pct(lat_miss, 0.99), n=len(lat_miss)),
        per_model_ms={f"{a}/{'hit' if h else 'miss'}": dict(p50=pct(v, 0.5), p99=pct(v, 0.99), n=len(v))
                      for (a, h), v in sorted(by_arch.items())},
        swap_gbps=(swap_bytes / 1e9) / (swap_ms * 1e-3) if swap_ms else None,
        pool_used_gib=st1["used"] / 2 ** 30, lru_models=st1["lru_models"],
    )


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--seconds", type=float, default=60.0)
    ap.add_argument("--rate", type=float, default=200.0)
    ap.add_argument("--caps-gb", type=float, nargs="+", default=[24.0, 8.0])
    ap.add_argument("--models", type=int, nargs=3, default=[32, 16, 16], metavar=("R50", "BERT", "R152"))
    args = ap.parse_args()

    from torpor_amd.server import Server

    runs = {}
    for cap in args.caps_gb:
        limit = int(cap * 2 ** 30)
        with Server(mem_limit_bytes=limit, pool_bytes=limit + (2 << 30)) as server:
            link = server.measure_h2d(256 << 20, 5)
            t0 = time.perf_counter()
            fleet = build_fleet(server, *args.models)
            reg_s = time.perf_counter() - t0
            charged = sum(server.model_info(f["fn"].fid)["total_bytes"] for f in fleet)
            weights = sum(server.model_info(f["fn"].fid)["image_bytes"] for f in fleet)
            r = serve(server, fleet, args.seconds, args.rate, seed=0)
            r.update(cap_gib=cap, cap_binds=charged >= limit, registration_s=reg_s,
                     charged_total_gib=charged / 2 ** 30, weights_total_gb=weights / 1e9, link_peak_gbps=link)
            runs[f"cap_{cap:g}GiB"] = r
            del fleet
    primary = runs[next(iter(runs))]
    print(json.dumps({
        "metric": "multi-tenant request latency p50 (ms), 64 models on 1 GPU, Poisson arrivals, Zipf(1.1) popularity",
        "value": primary["latency_ms"]["p50"], "unit": "ms", "n_gpus": 1, "higher_is_better": False,
        "dtype": "f32", "data": "synthetic (seeded random-init weights and inputs)",
        "config": {"workload": f"{args.models[0]}x ResNet-50 + {args.models[1]}x BERT-base s128 + "
                               f"{args.models[2]}x ResNet-152, batch 1, {args.rate:g} req/s, {args.seconds:g} s"},
        "runs": runs,
    }))


if __name__ == "__main__":
    main()
