#!/usr/bin/env python3
"""Cold-start benchmark of the model-swapping hot path on one MI355X.

A step is one cold request: Execute signal with the model swapped out -> layer-pipelined
swap-in overlapped with the forward pass -> logits in host memory, followed by the Unload that
makes the next step cold again (the reference's method, evaluation/table4/swap_pcie_latency/
test_scripts/swap_PCIe_latency.py:82-104).  Weights sit in the pinned host store and the request
input in host memory when the clock starts; nothing is resident in HBM.

One JSON line is printed: the headline value is the cold-start p50 of the primary workload,
BERT-large batch 4 seq 384 (BASELINE.json configs[3]: the largest single-GPU configuration and,
with ResNet-152, the one the north-star target is quoted on); the other single-GPU configs are
reported under "workloads".  "roofline" is computed from per-launch HIP-event timings of the
dominant kernel over timed warm requests, "swap" holds the swap-in GB/s (bytes that crossed the
link; compressible tensors travel in a lossless 27-bit format) against the measured pinned-host ->
HBM link peak, and "cpu_baseline" is the PyTorch CPU forward of the same
seeded model timed on this box's host cores (oracle/models.py, a reported baseline only).
"""
import argparse
import gc
import json
import os
import re
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
PEAK_HBM_GBPS = 8000.0          # MI355X HBM3E
PCIE_GEN5_X16_GBPS = 64.0       # nominal, per direction

WORKLOADS = {
    # name: (family, arch, batch, seq) - BASELINE.json configs[0..3]
    "resnet50-b1": ("resnet", "resnet50", 1, None),
    "bert-base-b1-s128": ("bert", "bert-base", 1, 128),
    "resnet152-b8": ("resnet", "resnet152", 8, None),
    "bert-large-b4-s384": ("bert", "bert-large", 4, 384),
}
PRIMARY = "bert-large-b4-s384"
# further served models (not part of the default run; `--workload <name>` measures one)
EXTRA_WORKLOADS = {
    "resnet101-b1": ("resnet", "resnet101", 1, None),
    "densenet169-b1": ("densenet", "densenet169", 1, None),
    "densenet201-b1": ("densenet", "densenet201", 1, None),
    "mobilenetv2-b1": ("mobilenet", "mobilenet_v2", 1, None),
    "efficientnet-b0-b1": ("efficientnet", "efficientnet_b0", 1, None),
    "inception-v3-b1": ("inception", "inception_v3", 1, None),
    "bert-large-qa-b1-s512": ("bert-qa", "bert-large", 1, 512),   # the reference endpoint's own call
}


def make_function(server, fid, name, seed=0):
    import torch
    from torpor_amd.functions import bert, densenet, efficientnet, inception, mobilenet, resnet

    family, arch, batch, seq = {**WORKLOADS, **EXTRA_WORKLOADS}[name]
    g = torch.Generator().manual_seed(0)
    if family == "densenet":
        weights = densenet.init_weights(arch, seed=seed)
        fn = densenet.DenseNet(server, fid, arch, batch=batch, weights=weights)
        inputs = [torch.randn(batch, 3, 224, 224, generator=g).numpy()]
    elif family == "inception":
        weights = inception.init_weights(seed=seed)
        fn = inception.InceptionV3(server, fid, batch=batch, weights=weights)
        inputs = [torch.randn(batch, 3, 299, 299, generator=g).numpy()]
    elif family == "efficientnet":
        weights = efficientnet.init_weights(seed=seed)
        fn = efficientnet.EfficientNetB0(server, fid, batch=batch, weights=weights)
        inputs = [torch.randn(batch, 3, 224, 224, generator=g).numpy()]
    elif family == "mobilenet":
        weights = mobilenet.init_weights(seed=seed)
        fn = mobilenet.MobileNetV2(server, fid, batch=batch, weights=weights)
        inputs = [torch.randn(batch, 3, 224, 224, generator=g).numpy()]
    elif family == "bert-qa":
        weights = bert.init_weights(arch, seed=seed, qa_head=True)
        fn = bert.Bert(server, fid, arch, batch=batch, seq=seq, weights=weights, token_types=True)
        inputs = [torch.randint(0, 30522, (batch, seq), generator=g).numpy(),
                  torch.randint(0, 2, (batch, seq), generator=g).numpy()]
    elif family == "resnet":
        weights = resnet.init_weights(arch, seed=seed)
        fn = resnet.ResNet(server, fid, arch, batch=batch, weights=weights)
        inputs = [torch.randn(batch, 3, 224, 224, generator=g).numpy()]
    else:
        weights = bert.init_weights(arch, seed=seed)
        fn = bert.Bert(server, fid, arch, batch=batch, seq=seq, weights=weights)
        inputs = [torch.randint(0, 30522, (batch, seq), generator=g).numpy()]
    return fn, inputs, weights


def pctl(xs, q):
    xs = sorted(xs)
    return xs[min(len(xs) - 1, int(round(q * (len(xs) - 1))))]


def run_workload(server, fid, name, steps, warmup, link_gbps):
    fn, inputs, weights = make_function(server, fid, name)
    first = fn.register(inputs)
    info = server.model_info(fid)
    packed, outbuf, views = fn.pack(inputs, pinned=True)   # results land in pinned memory, as a serving loop would have it

    def cold_step():
        fn.unload()
        t0 = time.perf_counter()
        ack, _, dfr = server.signal(1, fid, "")
        assert ack == 0 and not dfr
        server.replay(fid, packed, outbuf)
        return (time.perf_counter() - t0) * 1e3

    def warm_step():
        t0 = time.perf_counter()
        ack, _, dfr = server.signal(1, fid, "")
        assert ack == 0 and not dfr
        server.replay(fid, packed, outbuf)
        return (time.perf_counter() - t0) * 1e3

    for _ in range(warmup):
        cold_step()
    server.stream_synchronize(fid)
    gc.collect()
    gc.disable()   # as timeit does: a collection inside a timed step is the interpreter's, not the path's
    cold, swap_gbps, swap_ms = [], [], []
    t_begin = time.perf_counter()
    for _ in range(steps):
        cold.append(cold_step())
        st = server.swap_stats(fid)   # waits for the tail of the copy: part of the step
        swap_ms.append(st["copy_ms"])
        streams = st["copy_streams"]
        gathers = st["host_gathers"]
        swap_gbps.append(st["bytes"] / 1e9 / (st["copy_ms"] * 1e-3))   # bytes that crossed the link
        link_bytes = st["bytes"]
    server.stream_synchronize(fid)
    t_total = time.perf_counter() - t_begin
    out = fn.postprocess([v.copy() for v in views])
    for a, b in zip(first, out):
        if not np.array_equal(a, b):
            raise SystemExit(f"{name}: cold request output differs from the registration run")
    if not np.array_equal(server.readback_weights(fid), server.host_weights(fid)):
        raise SystemExit(f"{name}: swapped weights differ from the host copy")

    for _ in range(max(3, warmup)):
        warm_step()
    warm = [warm_step() for _ in range(max(steps, 20))]
    gc.enable()

    # per-kernel roofline accounting over timed warm requests
    server.profile_begin()
    nprof = 5
    for _ in range(nprof):
        warm_step()
    kstats, empty_us = server.profile_end()
    fn.unload()
    res = dict(
        cold_ms_p50=pctl(cold, 0.5), cold_ms_p99=pctl(cold, 0.99), cold_ms_min=min(cold),
        warm_ms_p50=pctl(warm, 0.5), warm_ms_min=min(warm),
        cold_over_warm=pctl(cold, 0.5) / pctl(warm, 0.5),
        exposed_swap_ms=pctl(cold, 0.5) - pctl(warm, 0.5),   # the part of the swap-in that compute did not hide
        weight_bytes=info["image_bytes"], act_bytes=info["act_bytes"], ops=info["n_ops"], chunks=info["n_chunks"],
        swap_ms_p50=pctl(swap_ms, 0.5), swap_gbps_p50=pctl(swap_gbps, 0.5),
        swap_frac_of_link=pctl(swap_gbps, 0.5) / link_gbps if link_gbps else None,
        link_bytes=link_bytes,   # below weight_bytes when tensors travel in the packed format
        weights_gbps_p50=info["image_bytes"] / 1e9 / (pctl(swap_ms, 0.5) * 1e-3),   # weight bytes in place per second
        copy_streams=streams, host_gathers=gathers, steps_total_s=t_total,
    )
    return res, kstats, empty_us, (fn, inputs, weights, first)


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` in `workload`, from the committed rocprofv3 --pmc summary
    (FETCH_SIZE and WRITE_SIZE runs of this same script, scaled by the copy-kernel calibration
    stated in that file); None when no summary covers this workload / kernel."""
    path = os.path.join(ROOT, "profiles", workload.replace("-", "_") + "_pmc_traffic.md")
    try:
        text = open(path).read()
    except OSError:
        return None
    m = re.search(r"^traffic_bytes_per_launch\[" + re.escape(kernel) + r"\]:\s*(\d+)", text, re.M)
    return int(m.group(1)) if m else None


def roofline_from(kstats, empty_us, workload):
    """Dominant kernel = largest summed duration; achieved = algorithmic work / time."""
    if not kstats:
        return None
    name, st = max(kstats.items(), key=lambda kv: kv[1]["total_us"])
    traffic = measured_traffic(workload, name)
    n = st["launches"]
    t_us = max(st["total_us"] - n * empty_us, 1e-3)
    avg_us = t_us / n
    if st["flops"] > 0:
        ach = st["flops"] / (t_us * 1e-6) / 1e12
        return dict(kernel=name, bound="mfma", achieved=ach, peak=PEAK_FP32_MFMA_TFLOPS, unit="TFLOP/s",
                    frac=ach / PEAK_FP32_MFMA_TFLOPS, traffic=traffic, launches=n, avg_launch_us=avg_us,
                    event_overhead_us=empty_us, flop_per_launch=st["flops"] / n, bytes_per_launch=st["bytes"] / n,
                    hbm_gbps=st["bytes"] / (t_us * 1e-6) / 1e9)
    ach = st["bytes"] / (t_us * 1e-6) / 1e9
    return dict(kernel=name, bound="hbm", achieved=ach, peak=PEAK_HBM_GBPS, unit="GB/s", frac=ach / PEAK_HBM_GBPS,
                traffic=traffic, launches=n, avg_launch_us=avg_us, event_overhead_us=empty_us,
                bytes_per_launch=st["bytes"] / n)


def cpu_baseline(name, weights, inputs, first):
    """PyTorch CPU forward of the same seeded model on this box's host cores."""
    import torch
    from oracle import models as om
    from torpor_amd.functions import bert

    family, arch, batch, seq = {**WORKLOADS, **EXTRA_WORKLOADS}[name]
    cores = int(os.environ.get("OMP_NUM_THREADS") or torch.get_num_threads())
    torch.set_num_threads(cores)
    if family in ("resnet", "densenet", "mobilenet", "efficientnet", "inception"):
        net = {"resnet": lambda: om.ResNet(arch), "densenet": lambda: om.DenseNet(arch),
               "mobilenet": lambda: om.MobileNetV2(), "efficientnet": lambda: om.EfficientNetB0(),
               "inception": lambda: om.InceptionV3()}[family]()
        model = om.load_numpy_state(net, weights)
        x = torch.from_numpy(inputs[0])
        fwd = lambda: (model(x),)
    elif family == "bert-qa":
        model = om.load_numpy_state(om.Bert(qa_head=True, **bert.CONFIGS[arch]), weights)
        x, tt = torch.from_numpy(inputs[0]), torch.from_numpy(inputs[1])
        fwd = lambda: model(x, tt)
    else:
        model = om.load_numpy_state(om.Bert(**bert.CONFIGS[arch]), weights)
        x = torch.from_numpy(inputs[0])
        fwd = lambda: model(x)
    times = []
    with torch.no_grad():
        for _ in range(3):
            out = fwd()
        for _ in range(10):
            t0 = time.perf_counter()
            out = fwd()
            times.append((time.perf_counter() - t0) * 1e3)
    err = 0.0
    for a, b in zip(first, out):
        b = b.numpy()
        err = max(err, float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)))
    return dict(value=statistics.median(times), unit="ms", cores=cores, kind="port",
                sample=f"10 timed forwards after 3 warm-ups of {name} (oracle/models.py, torch CPU fp32)",
                min_ms=min(times), logits_rel_err_vs_gpu=err)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="all", help="all | " + " | ".join(list(WORKLOADS) + list(EXTRA_WORKLOADS)))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--chunk-bytes", type=int, default=0)
    ap.add_argument("--chunk-max-bytes", type=int, default=0)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build serves from one GPU (one executor, one pool, one LRU per GPU); "
              "--gpus N with N > 1 is not supported", file=sys.stderr)
        sys.exit(2)

    from torpor_amd.server import Server

    names = list(WORKLOADS) if args.workload == "all" else [args.workload]
    if PRIMARY not in names:
        primary = names[0]
    else:
        primary = PRIMARY
    server = Server(mem_limit_bytes=24 << 30, pool_bytes=25 << 30, chunk_bytes=args.chunk_bytes,
                    chunk_max_bytes=args.chunk_max_bytes)
    link = server.measure_h2d(256 << 20, 10)
    results, roof, keep = {}, {}, {}
    for fid, name in enumerate(names):
        res, kstats, empty_us, ctx = run_workload(server, fid, name, args.steps, args.warmup, link)
        results[name] = res
        roof[name] = roofline_from(kstats, empty_us, name)
        res["kernels"] = {k: dict(launches=v["launches"], avg_us=max(v["total_us"] / v["launches"] - empty_us, 0.0),
                                  tflops=(v["flops"] / max(v["total_us"] - v["launches"] * empty_us, 1e-3) / 1e6),
                                  gbps=(v["bytes"] / max(v["total_us"] - v["launches"] * empty_us, 1e-3) / 1e3))
                          for k, v in sorted(kstats.items(), key=lambda kv: -kv[1]["total_us"])}
        if name == primary:
            keep = ctx
        else:
            del ctx
    cpu = None
    if not args.no_cpu:
        fn, inputs, weights, first = keep
        cpu = cpu_baseline(primary, weights, inputs, first)
    p = results[primary]
    line = {
        "metric": "cold-start latency p50 (swap-in + infer, ms) and swap-in GB/s vs link peak, 1 GPU",
        "value": p["cold_ms_p50"],
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": p["steps_total_s"] * 1e3 / args.steps,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (seeded random-init weights, seeded inputs)",
        "config": {"workload": primary + " fp32, weights in pinned host store, not resident in HBM at start"},
        "swap": {"gbps": p["swap_gbps_p50"], "link_peak_gbps_measured": link,
                 "frac_of_measured_link": p["swap_frac_of_link"], "pcie_gen5_x16_nominal_gbps": PCIE_GEN5_X16_GBPS,
                 "weight_bytes": p["weight_bytes"], "link_bytes": p["link_bytes"],
                 "weights_in_place_gbps": p["weights_gbps_p50"]},
        "warm_ms_p50": p["warm_ms_p50"],
        "cold_over_warm": p["cold_over_warm"],
        "roofline": roof[primary],
        "cpu_baseline": cpu,
        "workloads": results,
        "rooflines": roof,
    }
    server.close()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
