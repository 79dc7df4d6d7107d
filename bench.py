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
"link_roofline" prices the cold start against the host link: the bytes the request has to wait for
divided by the measured (and the nominal) link rate.  workloads["multitenant-64"] is a short leg of the
64-model configuration (BASELINE.json configs[4]) under its own 24 GiB cap and under a cap that binds.
`--ablate` adds the reference's pipeline ablation (evaluation/figure7/Figure7_README.md:12-33).
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
    "vgg16-b1": ("vgg", "vgg16", 1, None),
    "squeezenet1_1-b1": ("squeezenet", "squeezenet1_1", 1, None),
}


def make_function(server, fid, name, seed=0):
    import torch
    from torpor_amd.functions import bert, densenet, efficientnet, inception, mobilenet, resnet, squeezenet, vgg

    family, arch, batch, seq = {**WORKLOADS, **EXTRA_WORKLOADS}[name]
    g = torch.Generator().manual_seed(0)
    if family == "vgg":
        weights = vgg.init_weights(seed=seed)
        fn = vgg.VGG16(server, fid, batch=batch, weights=weights)
        inputs = [torch.randn(batch, 3, 224, 224, generator=g).numpy()]
    elif family == "squeezenet":
        weights = squeezenet.init_weights(seed=seed)
        fn = squeezenet.SqueezeNet11(server, fid, batch=batch, weights=weights)
        inputs = [torch.randn(batch, 3, 224, 224, generator=g).numpy()]
    elif family == "densenet":
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
        deferred_bytes = st["deferred_bytes"]
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
        input_bytes=int(packed.nbytes),   # the request's input crosses the link as well
        deferred_link_bytes=deferred_bytes,   # of those: index-looked-up tables, which travel last; the request does not wait for them
        weights_gbps_p50=info["image_bytes"] / 1e9 / (pctl(swap_ms, 0.5) * 1e-3),   # weight bytes in place per second
        copy_streams=streams, host_gathers=gathers, steps_total_s=t_total,
    )
    return res, kstats, empty_us, (fn, inputs, weights, first)


def measured_traffic(workload, kernel):
    """(HBM bytes per launch of `kernel` in `workload`, file) from the committed rocprofv3 --pmc summary
    (FETCH_SIZE and WRITE_SIZE runs of this same script, scaled by the copy-kernel calibration stated in
    that file); (None, None) when no summary covers this workload / kernel.  It is a figure read from that
    file, not a counter of this run: counters need the profiler."""
    rel = os.path.join("profiles", workload.replace("-", "_") + "_pmc_traffic.md")
    try:
        text = open(os.path.join(ROOT, rel)).read()
    except OSError:
        return None, None
    m = re.search(r"^traffic_bytes_per_launch\[" + re.escape(kernel) + r"\]:\s*(\d+)", text, re.M)
    return (int(m.group(1)), rel) if m else (None, None)


def profiled_average(workload, kernel):
    """(average duration in us of `kernel` over ALL its launches of one run of this workload's bench command
    under rocprofv3 --kernel-trace --stats, file) from the committed summary; (None, None) when none covers it.
    Unlike the event brackets, that average includes the launches of cold requests, which share the device with
    the swap-in's copies and unpack kernels."""
    rel = os.path.join("profiles", workload.replace("-", "_") + "_kernel_stats.md")
    try:
        text = open(os.path.join(ROOT, rel)).read()
    except OSError:
        return None, None
    m = re.search(r"^rocprof_avg_us\[" + re.escape(kernel) + r"\]:\s*([0-9.]+)", text, re.M)
    return (float(m.group(1)), rel) if m else (None, None)


def by_symbol(kstats):
    """{kernel symbol: summed stats + {shape: stats}} from the per-shape records of the engine
    (names are `symbol[shape]` for GEMM and convolution launches)."""
    out = {}
    for name, st in kstats.items():
        sym, _, shape = name.partition("[")
        e = out.setdefault(sym, dict(launches=0, total_us=0.0, flops=0.0, bytes=0.0, shapes={}))
        for k in ("launches", "total_us", "flops", "bytes"):
            e[k] += st[k]
        if shape:
            e["shapes"][shape.rstrip("]")] = st
    return out


def roofline_from(kstats, empty_us, workload):
    """Dominant kernel = the symbol with the largest summed duration; achieved = algorithmic work / time,
    per launch durations from HIP events around every launch on the compute stream, minus the duration of
    an empty event bracket."""
    if not kstats:
        return None
    syms = by_symbol(kstats)
    name, st = max(syms.items(), key=lambda kv: kv[1]["total_us"])
    traffic, traffic_file = measured_traffic(workload, name)
    n = st["launches"]
    t_us = max(st["total_us"] - n * empty_us, 1e-3)
    avg_us = t_us / n
    mfma = st["flops"] > 0
    ach = st["flops"] / (t_us * 1e-6) / 1e12 if mfma else st["bytes"] / (t_us * 1e-6) / 1e9
    peak = PEAK_FP32_MFMA_TFLOPS if mfma else PEAK_HBM_GBPS
    shapes = {}
    for shape, ss in sorted(st["shapes"].items(), key=lambda kv: -kv[1]["total_us"]):
        tt = max(ss["total_us"] - ss["launches"] * empty_us, 1e-3)
        a = ss["flops"] / (tt * 1e-6) / 1e12 if mfma else ss["bytes"] / (tt * 1e-6) / 1e9
        shapes[shape] = dict(launches=ss["launches"], avg_launch_us=tt / ss["launches"], achieved=a, frac=a / peak)
    r = dict(kernel=name, bound="mfma" if mfma else "hbm", achieved=ach, peak=peak, unit="TFLOP/s" if mfma else "GB/s",
             frac=ach / peak, traffic=traffic,
             traffic_source=(traffic_file + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command; read "
                             "from that file, not counted in this run)") if traffic_file else None,
             launches=n, avg_launch_us=avg_us, event_overhead_us=empty_us, bytes_per_launch=st["bytes"] / n,
             timing="frac, achieved, avg_launch_us: HIP-event brackets around each launch of 5 warm requests in "
                    "this run; frac_rocprof, rocprof_avg_launch_us: rocprofv3 --kernel-trace --stats average over "
                    "all launches of a run of this command (cold requests included), read from rocprof_source",
             by_shape=shapes)
    if mfma:
        r.update(flop_per_launch=st["flops"] / n, hbm_gbps=st["bytes"] / (t_us * 1e-6) / 1e9)
    prof_us, prof_file = profiled_average(workload, name)
    if prof_us:
        work = st["flops"] / n / 1e12 if mfma else st["bytes"] / n / 1e9
        r.update(rocprof_avg_launch_us=prof_us, frac_rocprof=work / (prof_us * 1e-6) / peak, rocprof_source=prof_file)
    return r


def link_roofline(res, link_gbps):
    """The cold start against the host link.  A request cannot answer before the bytes it needs have
    crossed the link: floor = (weight bytes on the link - tables that travel last + the request's own input,
    which goes the same way over the same link) / link rate."""
    waited = res["link_bytes"] - res["deferred_link_bytes"] + res.get("input_bytes", 0)
    floor_meas = waited / (link_gbps * 1e9) * 1e3
    floor_nom = waited / (PCIE_GEN5_X16_GBPS * 1e9) * 1e3
    return dict(bound="host link", bytes_waited_for=waited, input_bytes=res.get("input_bytes", 0), link_bytes=res["link_bytes"], weight_bytes=res["weight_bytes"],
                cold_ms_p50=res["cold_ms_p50"], floor_ms_at_measured_link=floor_meas,
                frac_of_measured_link_floor=floor_meas / res["cold_ms_p50"],
                floor_ms_at_nominal_64=floor_nom, frac_of_nominal_floor=floor_nom / res["cold_ms_p50"],
                full_image_floor_ms_at_measured_link=res["weight_bytes"] / (link_gbps * 1e9) * 1e3,
                # cold <= 1.3 x warm would need at most this many bytes over the measured link:
                bytes_for_1p3x_warm=1.3 * res["warm_ms_p50"] * 1e-3 * link_gbps * 1e9,
                # ... which is this many bits per 32-bit weight word the request waits for (the transfer
                # format sends 32 * link_bytes / weight_bytes of them today)
                bits_per_weight_word_for_1p3x_warm=32.0 * res["link_bytes"] / res["weight_bytes"] *
                                                   (1.3 * res["warm_ms_p50"] * 1e-3 * link_gbps * 1e9) / max(waited, 1))


def cpu_baseline(name, weights, inputs, first):
    """PyTorch CPU forward of the same seeded model on this box's host cores."""
    import torch
    from oracle import models as om
    from torpor_amd.functions import bert

    family, arch, batch, seq = {**WORKLOADS, **EXTRA_WORKLOADS}[name]
    cores = host_cores()
    torch.set_num_threads(cores)
    if family in ("resnet", "densenet", "mobilenet", "efficientnet", "inception", "vgg", "squeezenet"):
        net = {"resnet": lambda: om.ResNet(arch), "densenet": lambda: om.DenseNet(arch),
               "vgg": lambda: om.VGG16(), "squeezenet": lambda: om.SqueezeNet11(),
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
    return dict(value=statistics.median(times), unit="ms", cores=cores, kind="port", cpu=cpu_model_name(),
                os_cpu_count=os.cpu_count(),
                sample=f"10 timed forwards after 3 warm-ups of {name} (oracle/models.py, torch CPU fp32)",
                min_ms=min(times), logits_rel_err_vs_gpu=err)


def host_cores():
    """Host threads for the CPU leg: every core this process may run on (the scheduler's affinity mask where
    the platform has one, else os.cpu_count()), unless OMP_NUM_THREADS names the box's share explicitly."""
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit() and int(env) > 0:
        return int(env)
    try:
        return len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        return os.cpu_count() or 1


def cpu_model_name():
    try:
        for ln in open("/proc/cpuinfo"):
            if ln.startswith("model name"):
                return ln.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


ABLATION_VARIANTS = {
    "default": {},
    "group_per_tensor (BUFFER_SIZE=1)": dict(chunk_bytes=1, chunk_max_bytes=1),
    "one_group (no pipelining)": dict(chunk_bytes=2 << 30, chunk_max_bytes=2 << 30),
    "fixed_2MiB_groups (the reference's default)": dict(chunk_bytes=2 << 20, chunk_max_bytes=2 << 20),
    "weights_sent_as_they_are (TORPOR_PACK=0)": dict(pack=False),
    "lookups_wait_for_their_table (TORPOR_HOST_GATHER=0)": dict(host_gather=False),
}


def ablation_variant(vname, names, steps, warmup):
    """One variant of the ablation: one engine with that setting, the workloads one after the other on it, as in
    the main leg.  Cold p50 (ms), transfer groups, link bytes and swap-in GB/s per workload."""
    from torpor_amd.server import Server

    row = {}
    with Server(mem_limit_bytes=24 << 30, pool_bytes=25 << 30, **ABLATION_VARIANTS[vname]) as server:
        server.measure_h2d(256 << 20, 10)
        for fid, name in enumerate(names):
            fn, inputs, _ = make_function(server, fid, name)
            first = fn.register(inputs)
            packed, outbuf, views = fn.pack(inputs, pinned=True)
            cold = []
            for i in range(warmup + steps):
                fn.unload()
                t0 = time.perf_counter()
                ack, _, dfr = server.signal(1, fid, "")
                assert ack == 0 and not dfr
                server.replay(fid, packed, outbuf)
                if i >= warmup:
                    cold.append((time.perf_counter() - t0) * 1e3)
                st = server.swap_stats(fid)
            out_now = fn.postprocess([v.copy() for v in views])
            for a, b in zip(first, out_now):
                if not np.array_equal(a, b):
                    raise SystemExit(f"ablation {vname} / {name}: output differs from the registration run")
            row[name] = dict(cold_ms_p50=pctl(cold, 0.5), groups=st["chunks"], link_bytes=st["bytes"],
                             swap_gbps=st["bytes"] / 1e9 / (st["copy_ms"] * 1e-3))
            fn.unload()
            del fn
    return row


def ablation(names, steps, warmup):
    """Cold p50 (ms) per workload under the reference's pipeline ablation (evaluation/figure7/Figure7_README.md:
    12-33: BUFFER_SIZE = 2 MiB default, 1 = a group per tensor, 1.6 GB = no pipelining) and with this build's two
    own transfer features switched off.  These are engine settings, so every variant is an engine of its own --
    and a process of its own: the second and later engines of one process were measured with swap-ins of the small
    models at 40 instead of 55 GB/s (an engine's teardown frees tens of GiB of device memory, and copies that
    follow large frees run slower; a serving process has one engine and never frees device memory on the request
    path), which would be charged to the variant."""
    import subprocess

    out = {}
    for vname in ABLATION_VARIANTS:
        cmd = [sys.executable, os.path.abspath(__file__), "--ablation-variant", vname, "--steps", str(steps),
               "--warmup", str(warmup), "--workload", "all" if len(names) > 1 else names[0]]
        r = subprocess.run(cmd, capture_output=True, text=True, timeout=900)
        if r.returncode != 0:
            raise SystemExit(f"bench.py: ablation variant {vname!r} failed:\n{r.stderr[-2000:]}")
        out[vname] = json.loads(r.stdout.strip().splitlines()[-1])
    return out


CAL_COPY_BYTES = 64 << 20


def counter_calibration_copy(server, fid=65000, repeats=3):
    """Plain device-to-device copies of known size (64 MiB read and 64 MiB written each, far beyond the L2s) by
    the library's `copy_kernel`: what the FETCH_SIZE / WRITE_SIZE counters of a profiled run of this command are
    scaled by.  A scratch function of its own, registered, run once and unloaded; a few milliseconds."""
    import numpy as np

    from torpor_amd.server import OP_FILL, REQ_EXECUTE_AFTER_LOAD, REQ_UNLOAD
    ack, _, deferred = server.signal(REQ_EXECUTE_AFTER_LOAD, fid, "1")
    assert ack == 0 and not deferred
    w = np.zeros(4, np.float32)
    server.h2d(fid, server.malloc(fid, w.nbytes), w)
    server.device_synchronize(fid)                      # end of the loading phase
    src, dst = server.malloc(fid, CAL_COPY_BYTES), server.malloc(fid, CAL_COPY_BYTES)
    server.memset(fid, src, 0, CAL_COPY_BYTES)
    for _ in range(repeats):
        server.d2d(fid, dst, src, CAL_COPY_BYTES)
    done = server.malloc(fid, 4)                        # the request ends with its device-to-host copy
    server.launch(fid, OP_FILL, [done], [1], [0.0])
    out = np.empty(1, np.float32)                       # alive until the synchronisation has delivered it
    server.d2h_async(fid, out, done)
    server.stream_synchronize(fid)
    server.signal(REQ_UNLOAD, fid, "")


COMPACT_LIMIT_BYTES = 6000   # the final stdout line stays below this; everything else goes to the detail file


def sig(x, digits=4):
    """Floats to `digits` significant figures (the line is read by programs and people, not re-used in arithmetic)."""
    if isinstance(x, bool) or not isinstance(x, float):
        return x
    if x != x or x in (float("inf"), float("-inf")):
        return None
    return float(f"{x:.{digits}g}")


def trim(obj, digits=4):
    if isinstance(obj, dict):
        return {k: trim(v, digits) for k, v in obj.items()}
    if isinstance(obj, (list, tuple)):
        return [trim(v, digits) for v in obj]
    if isinstance(obj, (np.floating,)):
        return sig(float(obj), digits)
    if isinstance(obj, (np.integer,)):
        return int(obj)
    return sig(obj, digits)


def compact_roofline(r):
    """The roofline object without its per-shape table and prose."""
    if not r:
        return None
    keep = ("kernel", "bound", "achieved", "peak", "unit", "frac", "traffic", "launches", "avg_launch_us",
            "flop_per_launch", "bytes_per_launch", "frac_rocprof", "rocprof_avg_launch_us")
    out = {k: r[k] for k in keep if k in r}
    if "frac_rocprof" in out:
        out["timing"] = "frac: HIP-event brackets, warm requests, this run; frac_rocprof: rocprofv3 average, all launches, " + r["rocprof_source"]
    else:
        out["timing"] = "frac: HIP-event brackets, warm requests, this run"
    if r.get("traffic") and r.get("bytes_per_launch"):
        out["traffic_over_algorithmic"] = r["traffic"] / r["bytes_per_launch"]
    return out


def compact_line(line, detail_path=None):
    """The one JSON line a driver parses: the headline, its roofline / link roofline / CPU baseline, one short
    record per workload and a few numbers per multi-tenant run.  Per-shape tables, per-kernel lists, per-model
    percentiles and the ablation live in the detail file."""
    out = {k: line[k] for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                                "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "swap",
                                "warm_ms_p50", "cold_over_warm") if k in line}
    out["roofline"] = compact_roofline(line.get("roofline"))
    lr = line.get("link_roofline") or {}
    out["link_roofline"] = {k: lr[k] for k in ("bound", "bytes_waited_for", "floor_ms_at_measured_link",
                                               "frac_of_measured_link_floor", "floor_ms_at_nominal_64") if k in lr} or None
    cpu = line.get("cpu_baseline")
    out["cpu_baseline"] = ({k: cpu[k] for k in ("value", "unit", "cores", "kind", "sample", "cpu", "os_cpu_count",
                                                "logits_rel_err_vs_gpu") if k in cpu} if cpu else None)
    wl = {}
    for name, res in (line.get("workloads") or {}).items():
        if name == "multitenant-64":
            continue
        roof = (line.get("rooflines") or {}).get(name) or {}
        lrw = res.get("link_roofline") or {}
        wl[name] = dict(cold_ms_p50=res["cold_ms_p50"], warm_ms_p50=res["warm_ms_p50"],
                        cold_over_warm=res["cold_over_warm"], swap_gbps=res["swap_gbps_p50"],
                        frac_of_link=res["swap_frac_of_link"], cold_over_link_floor=(
                            1.0 / lrw["frac_of_measured_link_floor"] if lrw.get("frac_of_measured_link_floor") else None),
                        launches=res.get("ops"), kernel=roof.get("kernel"), frac=roof.get("frac"),
                        avg_launch_us=roof.get("avg_launch_us"))
    out["workloads"] = wl
    mt = ((line.get("workloads") or {}).get("multitenant-64") or {}).get("runs") or {}
    if mt:
        out["multitenant"] = {
            run: dict(seconds=r.get("wall_s"), dispatch=r.get("dispatch"), hit_ratio=r["hit_ratio"],
                      p50_ms=r["latency_ms"]["p50"], p99_ms=r["latency_ms"]["p99"], hit_p50_ms=r["hit_ms"]["p50"],
                      hit_p99_ms=r["hit_ms"]["p99"], miss_p50_ms=r["miss_ms"]["p50"], swap_gbps=r.get("swap_gbps"))
            for run, r in mt.items()}
    if detail_path:
        out["detail"] = detail_path
    out = trim(out)
    # never let the line outgrow what the driver reads: drop the optional blocks, largest first
    for victim in ("multitenant", "workloads", "link_roofline"):
        if len(json.dumps(out, separators=(",", ":"))) <= COMPACT_LIMIT_BYTES:
            break
        out.pop(victim, None)
    return out


def write_detail(line, path=None):
    """Everything measured, as indented JSON beside the other run outputs; returns the path written (relative to the
    repository) or None when the directory cannot be written."""
    path = path or os.path.join(ROOT, "gpurun_out", "bench_detail.json")
    try:
        os.makedirs(os.path.dirname(path), exist_ok=True)
        with open(path, "w") as f:
            json.dump(trim(line, 6), f, indent=1)
    except OSError as e:
        print(f"bench.py: detail file not written: {e}", file=sys.stderr)
        return None
    return os.path.relpath(path, ROOT)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="all", help="all | " + " | ".join(list(WORKLOADS) + list(EXTRA_WORKLOADS)))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--chunk-bytes", type=int, default=0)
    ap.add_argument("--chunk-max-bytes", type=int, default=0)
    ap.add_argument("--no-multitenant", action="store_true", help="skip the 64-model leg")
    ap.add_argument("--multitenant-seconds", type=float, default=60.0)
    ap.add_argument("--multitenant-caps-gb", type=float, nargs="+", default=[24.0, 8.0])
    ap.add_argument("--ablate", action="store_true",
                    help="also measure cold p50 per config with per-tensor groups, one whole-image group, weights "
                         "sent as they are, and lookups that wait for their table")
    ap.add_argument("--ablation-variant", default=None, help=argparse.SUPPRESS)   # child of --ablate
    ap.add_argument("--detail", default=None, help="where the full results go (default gpurun_out/bench_detail.json)")
    args = ap.parse_args()
    import __graft_entry__
    __graft_entry__.ensure_built()      # a fresh checkout is compiled first; a built tree is used as it is
    if args.ablation_variant is not None:
        names = list(WORKLOADS) if args.workload == "all" else [args.workload]
        print(json.dumps(ablation_variant(args.ablation_variant, names, args.steps, args.warmup)))
        return
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
    counter_calibration_copy(server)
    results, roof, keep = {}, {}, {}
    for fid, name in enumerate(names):
        res, kstats, empty_us, ctx = run_workload(server, fid, name, args.steps, args.warmup, link)
        results[name] = res
        roof[name] = roofline_from(kstats, empty_us, name)
        res["kernels"] = {k: dict(launches=v["launches"], avg_us=max(v["total_us"] / v["launches"] - empty_us, 0.0),
                                  tflops=(v["flops"] / max(v["total_us"] - v["launches"] * empty_us, 1e-3) / 1e6),
                                  gbps=(v["bytes"] / max(v["total_us"] - v["launches"] * empty_us, 1e-3) / 1e3))
                          for k, v in sorted(kstats.items(), key=lambda kv: -kv[1]["total_us"])}
        res["link_roofline"] = link_roofline(res, link)
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
        "link_roofline": p.get("link_roofline"),
        "cpu_baseline": cpu,
        "workloads": results,
        "rooflines": roof,
    }
    server.close()
    if args.workload == "all" and not args.no_multitenant:
        from torpor_amd import multitenant as mt
        runs = {}
        tight = min(args.multitenant_caps_gb)
        for cap in args.multitenant_caps_gb:
            # the configuration's own cap does not bind (nothing is ever swapped): a short run; the cap that binds
            # gets the full length, served through the miss-aware dispatcher (torpor_amd/dispatch.py)
            secs = args.multitenant_seconds if cap == tight else min(args.multitenant_seconds, 10.0)
            runs[f"cap_{cap:g}GiB"] = mt.run_cap(cap, secs, 200.0, dispatch="miss-aware")
        # the binding cap once more on the same trace in arrival order, as the reference's router hands requests over
        runs[f"cap_{tight:g}GiB_in_order"] = mt.run_cap(tight, args.multitenant_seconds, 200.0, dispatch="in-order")
        line["workloads"]["multitenant-64"] = dict(
            config="32x ResNet-50 + 16x BERT-base s128 + 16x ResNet-152, seeds 0..63, batch 1, open-loop Poisson "
                   f"200 req/s, Zipf(1.1) popularity, {args.multitenant_seconds:g} s under the binding cap; "
                   "latency = completion - arrival",
            runs=runs)
    if args.ablate:
        line["ablation"] = ablation(names, max(args.steps // 2, 5), max(args.warmup, 8))
    detail_path = write_detail(line, args.detail)
    print(json.dumps(compact_line(line, detail_path), separators=(",", ":")))


if __name__ == "__main__":
    main()
