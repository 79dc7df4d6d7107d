"""The final stdout line of bench.py is what the driver parses: it has to stay small, be strict JSON and carry the
headline, `roofline` and `cpu_baseline`, whatever the run measured beside them."""
import json
import math

import bench


def kernel_stats(n_shapes):
    return {f"gemm_fast_64x32_kc_s2[{1536 + i}x1024x4096]": dict(launches=24, total_us=2700.0 + i, flops=3.1e11, bytes=1.2e9)
            for i in range(n_shapes)}


def workload_result(i):
    res = dict(cold_ms_p50=18.7 + i, cold_ms_p99=19.1, cold_ms_min=18.5, warm_ms_p50=9.4 / 3, warm_ms_min=9.3,
               cold_over_warm=1.98765432101, exposed_swap_ms=9.3, weight_bytes=1340567552, act_bytes=123456789, ops=173,
               chunks=86, swap_ms_p50=20.1, swap_gbps_p50=56.3333333, swap_frac_of_link=0.98, link_bytes=1138963712,
               deferred_link_bytes=106210048, weights_gbps_p50=66.1, copy_streams=2, host_gathers=1, steps_total_s=0.41)
    res["kernels"] = {f"kernel_{k}[{k}x{k}x{k}]": dict(launches=5, avg_us=1.0 / 3, tflops=100.0 / 3, gbps=1e3 / 7)
                      for k in range(60)}
    res["link_roofline"] = bench.link_roofline(res, 57.1)
    return res


def multitenant_run():
    pm = {f"{a}/{h}": dict(p50=1.0 / 3, p99=7.0 / 3, n=100) for a in ("resnet50", "resnet152", "bert-base") for h in ("hit", "miss")}
    return dict(requests=12000, wall_s=60.1, achieved_rps=199.7, hit_ratio=0.87, evictions=1535, fragmentation_evictions=7,
                swap_ins=1546, lookahead=0, prefetches=0, dispatch="miss-aware",
                latency_ms=dict(p50=0.63, p99=7.28, mean=1.4), hit_ms=dict(p50=0.61, p99=2.9, n=10000),
                miss_ms=dict(p50=3.8, p99=9.0, n=1546), per_model_ms=pm, swap_gbps=55.8, pool_used_gib=7.98,
                lru_models=36, pinned_host_gib=12.6, device_outside_pool_gib=0.41, cap_gib=8.0, cap_binds=True,
                registration_s=18.0, offered_rps=200.0, charged_total_gib=13.97, weights_total_gb=14.15, link_peak_gbps=56.3)


def full_line(nan_somewhere=False):
    names = list(bench.WORKLOADS)
    results = {n: workload_result(i) for i, n in enumerate(names)}
    roof = {n: bench.roofline_from(kernel_stats(12), 4.3, n) for n in names}
    p = results[bench.PRIMARY]
    line = {"metric": "cold-start latency p50 (swap-in + infer, ms) and swap-in GB/s vs link peak, 1 GPU",
            "value": p["cold_ms_p50"], "unit": "ms", "n_gpus": 1, "steps": 20, "warmup": 5, "ms_per_step": 20.4,
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
            "data": "synthetic (seeded random-init weights, seeded inputs)",
            "config": {"workload": bench.PRIMARY + " fp32, weights in pinned host store, not resident in HBM at start"},
            "swap": {"gbps": 56.3, "link_peak_gbps_measured": 57.1, "frac_of_measured_link": 0.985,
                     "pcie_gen5_x16_nominal_gbps": 64.0, "weight_bytes": 1340567552, "link_bytes": 1138963712,
                     "weights_in_place_gbps": 66.3},
            "warm_ms_p50": p["warm_ms_p50"], "cold_over_warm": float("nan") if nan_somewhere else p["cold_over_warm"],
            "roofline": roof[bench.PRIMARY], "link_roofline": p["link_roofline"],
            "cpu_baseline": dict(value=814.1, unit="ms", cores=16, kind="port", cpu="some host cpu", os_cpu_count=256,
                                 sample="10 timed forwards after 3 warm-ups", min_ms=800.0, logits_rel_err_vs_gpu=3.1e-6),
            "workloads": results, "rooflines": roof}
    line["workloads"]["multitenant-64"] = dict(config="...", runs={f"cap_{c}": multitenant_run()
                                                                    for c in ("24GiB", "8GiB", "8GiB_in_order", "8GiB_lookahead1")})
    line["ablation"] = {v: {n: dict(cold_ms_p50=1.0, groups=3, link_bytes=5, swap_gbps=50.0) for n in names}
                        for v in bench.ABLATION_VARIANTS}
    return line


def strict_loads(text):
    def refuse(tok):
        raise ValueError(f"not strict JSON: {tok}")
    return json.loads(text, parse_constant=refuse)


def test_final_line_is_small_strict_json_with_the_required_objects():
    full = full_line()
    assert len(json.dumps(full)) > 20000            # the case that defeated the driver: the full record is large
    text = json.dumps(bench.compact_line(full, "gpurun_out/bench_detail.json"), separators=(",", ":"))
    assert "\n" not in text and len(text.encode()) <= bench.COMPACT_LIMIT_BYTES <= 6000
    line = strict_loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "swap", "cold_over_warm"):
        assert key in line, key
    assert set(line["config"]) == {"workload"}
    r = line["roofline"]
    assert r["bound"] in ("hbm", "mfma") and r["unit"] in ("GB/s", "TFLOP/s")
    assert math.isclose(r["frac"], r["achieved"] / r["peak"], rel_tol=2e-3)
    assert "by_shape" not in r and "traffic" in r
    c = line["cpu_baseline"]
    assert c["kind"] in ("port", "reference") and c["cores"] == 16 and c["value"] > 0 and c["sample"]
    assert set(line["workloads"]) == set(bench.WORKLOADS)
    assert all("kernels" not in w for w in line["workloads"].values())
    assert len(line["multitenant"]) == 4 and all("per_model_ms" not in r for r in line["multitenant"].values())
    assert line["detail"] == "gpurun_out/bench_detail.json"


def test_final_line_has_no_nan_and_sheds_optional_blocks_before_it_outgrows_the_limit():
    full = full_line(nan_somewhere=True)
    line = bench.compact_line(full)
    assert line["cold_over_warm"] is None
    strict_loads(json.dumps(line))
    # forty workloads would not fit: the optional blocks go, the required ones stay
    for i in range(40):
        full["workloads"][f"extra-{i}-with-a-long-name-to-take-up-room"] = workload_result(i)
    text = json.dumps(bench.compact_line(full), separators=(",", ":"))
    assert len(text.encode()) <= bench.COMPACT_LIMIT_BYTES
    line = strict_loads(text)
    assert line["roofline"] and line["cpu_baseline"] and line["value"]


def test_detail_file_holds_the_whole_record(tmp_path):
    full = full_line()
    path = bench.write_detail(full, str(tmp_path / "d" / "bench_detail.json"))
    assert path is not None
    back = strict_loads(open(tmp_path / "d" / "bench_detail.json").read())
    assert "by_shape" in back["roofline"] and "ablation" in back and "kernels" in back["workloads"][bench.PRIMARY]
    assert "per_model_ms" in back["workloads"]["multitenant-64"]["runs"]["cap_8GiB"]
