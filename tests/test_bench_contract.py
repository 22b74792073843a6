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
            ("quant_pack_int2_1000000x256", "quant_pack_rows_kernel"), ("unpack_dequant_int2_1000000x256", "unpack_dequant_rows_kernel"),
            ("quant_pack_int2_2000000x128", "quant_pack_rows_kernel"), ("quant_pack_int2_4000000x64", "quant_pack_rows_kernel"),
            ("quant_pack_int2_425000x602", "quant_pack_rows_kernel"), ("unpack_dequant_int2_425000x602", "unpack_dequant_rows_kernel"),
            ("prepost_8000000n_160000000ue_local_2000000c_80000000e_remote_int2_F128", "spmm_piece_kernel(dq)"),
            ("prepost_8000000n_160000000ue_local_2000000c_80000000e_remote_int2_F128", "spmm_piece_kernel(local)"),
            ("prepost_8000000n_160000000ue_local_2000000c_80000000e_remote_int2_F128", "spmm_short_kernel(local)")]
    for key in want:
        t = b.TRAFFIC.get(key)
        assert t is not None, f"no traffic line for {key} under profiles/"
        assert t["bytes"] == t["fetch_bytes"] + t["write_bytes"] > 0 and t["source"].startswith("profiles/")


def test_roofline_fraction_is_measured_traffic_over_time_over_peak():
    b = _bench()
    key = ("quant_pack_int2_1000000x256", "quant_pack_rows_kernel")
    t = b.TRAFFIC[key]
    r = b.roofline(key[0], key[1], kernel_ms=0.170, algorithmic_bytes=1_096_000_000)
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["traffic"] == t["bytes"]
    assert abs(r["achieved"] - t["bytes"] / 0.170 / 1e6) < 0.1 and abs(r["frac"] - r["achieved"] / 8000.0) < 1e-4 and r["frac"] <= 1.0
    assert abs(r["gather_model"]["GBps"] - 1_096_000_000 / 0.170 / 1e6) < 0.1
    none = b.roofline("no_such_workload", "k", 1.0, 10)        # nothing measured: no fraction is made up
    assert none["achieved"] is None and none["frac"] is None and none["traffic"] is None
