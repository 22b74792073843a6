"""bench.py's contract that can be checked without a GPU: it refuses more than one GPU, and the measured-traffic
figures its roofline objects divide by are present, for every workload of the default run, in the tracked
rocprofv3 summaries under profiles/."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_measured_traffic_of_every_default_workload_is_tracked():
    b = _bench()
    want = [("rmat_2450000n_62000000e_F128_gcn_weighted_sum", "spmm_piece_kernel"),
            ("rmat_2450000n_62000000e_F128_gcn_weighted_sum", "spmm_short_kernel"),
            ("rmat_2450000n_62000000e_F128_gcn_weighted_sum", "spmm_long_final_kernel"),
            ("sbm_233000n_113597648e_F602_sum", "spmm_band_kernel"),
            *[(f"{k}_int{b}_{shape}", f"{k}_rows_kernel") for k in ("quant_pack", "unpack_dequant") for b in (8, 4, 2)
              for shape in ("1000000x256", "2000000x128", "4000000x64", "425000x602", "2560000x100")],
            ("prepost_8000000n_160000000ue_local_2000000c_80000000e_remote_int2_F128", "spmm_piece_kernel(dq)"),
            ("prepost_8000000n_160000000ue_local_2000000c_80000000e_remote_int2_F128", "spmm_piece_kernel(local)"),
            ("prepost_8000000n_160000000ue_local_2000000c_80000000e_remote_int2_F128", "spmm_short_kernel(local)")]
    for key in want:
        t = b.TRAFFIC.get(key)
        assert t is not None, f"no traffic line for {key} under profiles/"
        assert t["bytes"] == t["fetch_bytes"] + t["write_bytes"] > 0 and t["source"].startswith("profiles/")
        if not key[0].startswith(("quant_pack", "unpack_dequant")):
            assert t["plan"], f"the traffic line of {key} does not say which plan shape it was measured on"


def test_roofline_fraction_is_measured_traffic_over_time_over_peak():
    b = _bench()
    key = ("quant_pack_int2_1000000x256", "quant_pack_rows_kernel")
    t = b.TRAFFIC[key]
    r = b.roofline(key[0], key[1], kernel_ms=0.170, algorithmic_bytes=1_096_000_000)
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["traffic"] == t["bytes"]
    assert abs(r["achieved"] - t["bytes"] / 0.170 / 1e6) < 0.1 and abs(r["frac"] - r["achieved"] / 8000.0) < 1e-4 and r["frac"] <= 1.0
    assert abs(r["gather_GBps"] - 1_096_000_000 / 0.170 / 1e6) < 0.1
    none = b.roofline("no_such_workload", "k", 1.0, 10)        # nothing measured: no fraction is made up
    assert none["achieved"] is None and none["frac"] is None and none["traffic"] is None


def _canned_results(b):
    """Result dicts shaped like the workloads' own, from made-up times."""
    wl = "rmat_2450000n_62000000e_F128_gcn_weighted_sum"
    head = {"metric": "SpMM GEdges/s + % HBM roofline (F=128 fp32); quantize-pack GB/s at int2", "value": 19.8123456, "unit": "GEdges/s",
            "config": {"workload": wl, "nodes": 2450000, "edges": 62000000, "F": 128, "aggregation": "weighted_sum",
                       "accumulate": True, "index_dtype": "int32"},
            "ms_per_step": 3.1298765, "dtype": "f32",
            "roofline": b.roofline(wl, "spmm_piece_kernel", 1.7236, 24_560_000_000, 1),
            "cpu_baseline": {"value": 0.41234567, "unit": "GEdges/s", "cores": 16, "host_cpu_count": 256, "kind": "reference",
                             "sample": "2450000 of 2450000 rows (62000000 edges) of the same graph, full X, F=128, 1 warm-up + median of 10",
                             "ms": 150.0},
            "extra": {"plan_build_ms": 131.6, "plan": {"long_rows": 97836, "pieces": 996264}, "empty_rows": 1029439,
                      "spmm_mean_GEdges_per_s": 20.123, "spmm_GFLOPs": 5071.2, "kernel_ms_per_step": {"spmm_piece_kernel": 1.7},
                      "kernel_rooflines": {"x": {"y": {"z": 1}}}, "edge_values_bound_to_plan": True}}
    others = {}
    for name, (n, F) in {"quant": (1_000_000, 256), "quant_F128": (2_000_000, 128), "quant_F64": (4_000_000, 64),
                         "quant_F602": (425_000, 602), "quant_F100": (2_560_000, 100)}.items():
        extra = {}
        for bits in (8, 4, 2):
            w = f"quant_pack_int{bits}_{n}x{F}"
            nb = b.quant_bytes(n, F, bits)
            extra[f"int{bits}"] = {"bytes": nb, "quant_ms": 0.2, "dequant_ms": 0.19,
                                   "quant_roofline": b.streaming_roofline(w, "quant_pack_rows_kernel", 0.17, nb),
                                   "dequant_roofline": b.streaming_roofline(w.replace("quant_pack", "unpack_dequant"),
                                                                            "unpack_dequant_rows_kernel", 0.16, nb)}
        others[name] = {"metric": "quantize-pack GB/s at int2", "value": 6000.0, "unit": "GB/s",
                        "config": {"workload": f"quant_pack_int2_{n}x{F}"}, "ms_per_step": 0.2, "dtype": "f32->u8",
                        "roofline": extra["int2"]["quant_roofline"], "cpu_baseline": None, "extra": extra}
    for name, kern in (("copy", "stream_copy_kernel"), ("sbm", "spmm_band_kernel"), ("prepost", "spmm_piece_kernel(dq)"),
                       ("small", "spmm_short_kernel")):
        others[name] = {"metric": "m" * 90, "value": 7.0123456, "unit": "GEdges/s", "config": {"workload": "w" * 70},
                        "ms_per_step": 16.2, "dtype": "f32", "roofline": b.roofline("sbm_233000n_113597648e_F602_sum", kern, 15.9, 1e11, 18),
                        "cpu_baseline": dict(head["cpu_baseline"]), "extra": {"schedule": {"band": 1}, "big": list(range(500))}}
    return head, others


def test_printed_line_is_small_flat_and_complete():
    """The line is built by the code path main() uses; it must stay far below what the reading harness keeps of
    stdout, and carry the roofline and CPU-baseline objects and the int2 quantize+pack figure of the metric."""
    import json
    b = _bench()
    head, others = _canned_results(b)
    text = b.build_line(head, others, 20, 5)
    assert "\n" not in text and len(text) < 4096, len(text)
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    r = line["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s" and 0 < r["frac"] <= 1.0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3 and r["traffic"] > 0 and r["kernel"] == "spmm_piece_kernel"
    c = line["cpu_baseline"]
    assert c["value"] > 0 and c["kind"] in ("reference", "port") and c["cores"] == 16 and "sample" in c
    assert line["config"]["workload"].startswith("rmat_") and line["vs_baseline"] is None and line["n_gpus"] == 1
    ex = line["extra"]
    assert ex["quant_pack_int2_GBps"] > 0 and 0 < ex["quant_pack_int2_frac"] <= 1.0
    # nothing nested below a workload's flat record
    for name, rec in ex["workloads"].items():
        assert all(not isinstance(v, (dict, list)) for v in rec.values()), name
    assert all(not isinstance(v, (dict, list)) for k, v in ex.items() if k != "workloads")
    assert {"sbm", "prepost", "small", "copy", "quant_int8", "quant_int4", "quant_int2", "quant_F602_int2"} <= set(ex["workloads"])
    assert ex["workloads"]["sbm"]["cpu"] > 0


def test_line_never_exceeds_the_limit_even_with_many_workloads():
    import json
    b = _bench()
    head, others = _canned_results(b)
    for i in range(60):
        others[f"more_{i}"] = dict(others["sbm"])
    text = b.build_line(head, others, 20, 5)
    assert len(text) <= b.LINE_LIMIT
    line = json.loads(text)
    assert line["roofline"]["frac"] and line["cpu_baseline"]["value"]


def test_traffic_measured_on_another_plan_gives_no_fraction():
    b = _bench()
    key = ("w_test", "k_test")
    b.TRAFFIC[key] = {"bytes": 10 ** 9, "fetch_bytes": 10 ** 9, "write_bytes": 0, "l2_hit": 0.5, "plan": "n_bands:18,n_slices:1",
                      "source": "profiles/x.txt"}
    same = b.roofline("w_test", "k_test", 1.0, 10 ** 9, plan=b.plan_signature(n_slices=1, n_bands=18))
    other = b.roofline("w_test", "k_test", 1.0, 10 ** 9, plan=b.plan_signature(n_slices=2, n_bands=9))
    assert same["frac"] == 0.125 and other["frac"] is None and other["traffic"] is None and other["gather_frac"] == 0.125
