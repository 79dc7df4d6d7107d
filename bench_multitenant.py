#!/usr/bin/env python3
"""Multi-tenant serving benchmark on one MI355X (BASELINE.json configs[4]), the long form of the leg that
bench.py reports under workloads["multitenant-64"].

64 random-init models (32 ResNet-50, 16 BERT-base seq 128, 16 ResNet-152; seeds 0..63, batch 1)
are registered, so all weights sit in the pinned host store; requests then arrive as an open-loop
Poisson process (default 200 req/s) with Zipf(1.1) popularity over the 64 functions (the arrival
process of the reference's load generator, scripts/sender_fix_rate.py:46-56) and are served by the
single executor, one active function at a time: --dispatch miss-aware (default; requests of resident
models run while the swap-in of the oldest swapped-out one streams, torpor_amd/dispatch.py) or in-order
(arrival order).  Latency = completion - arrival, so it includes queueing.

What the pool cap charges: per resident model, its weight image plus its activation arena, each
rounded up to 2 MiB slabs (the reference also charges every block of a model,
include/server/model_repo.hpp:139-140).  The 64 models total about 14 GiB charged, so the
24 GiB cap of the config does not force evictions; the run is therefore repeated with a binding
cap (default 8 GiB) and both are reported.

--lookahead N: when a request starts, the models of up to N requests already waiting behind it are
prefetched with Load requests (their swap-ins then overlap this request's compute).

Prints one JSON line.  Usage: python bench_multitenant.py [--seconds 60] [--rate 200] [--caps-gb 24 8] [--lookahead 1]
"""
import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--seconds", type=float, default=60.0)
    ap.add_argument("--rate", type=float, default=200.0)
    ap.add_argument("--caps-gb", type=float, nargs="+", default=[24.0, 8.0])
    ap.add_argument("--models", type=int, nargs=3, default=[32, 16, 16], metavar=("R50", "BERT", "R152"))
    ap.add_argument("--lookahead", type=int, default=0)
    ap.add_argument("--dispatch", choices=["in-order", "miss-aware"], default="miss-aware",
                    help="order in which arrived requests are handed to the executor (torpor_amd/dispatch.py)")
    args = ap.parse_args()

    from torpor_amd import multitenant as mt

    runs = {f"cap_{cap:g}GiB": mt.run_cap(cap, args.seconds, args.rate, models=tuple(args.models), lookahead=args.lookahead,
                                              dispatch=args.dispatch)
            for cap in args.caps_gb}
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
