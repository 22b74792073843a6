#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path over one batch of synthetic input that is already resident in
HBM: by default the headline configuration, a weighted-sum SpMM (out += A @ X, GCN-normalised edge
weights) over an R-MAT power-law graph with 2.45 M nodes / ~62 M stored edges at F = 128 fp32.
The same run also reports, as extras, the mean-aggregation variant, the int8/int4/int2
quantize+pack and unpack+dequantize kernels on 1 M x 256 boundary rows, a plain streaming copy (the
attainable-bandwidth yardstick), and a CPU baseline timed on this machine's host cores.

Prints ONE JSON line on stdout (everything else goes to stderr).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this file (see profiles/), scaled by what the same counters read for sgnn_stream_copy_f32 of a
# known size.  Keyed by workload name; None = not measured.
MEASURED_TRAFFIC_BYTES = {
    # spmm_piece_kernel (values bound to the plan): FETCH_SIZE 4041502 x 2.000 + WRITE_SIZE 860068 x 1.000 (KiB per launch)
    "rmat_2450000n_62000000e_F128_gcn_weighted_sum": 9_157_000_000,
    # quant_pack_rows16_kernel<2,...>: FETCH_SIZE 500052 x 2.000 + WRITE_SIZE 76196 x 1.000
    "quant_pack_int2_1000000x256": 1_102_000_000,
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def spmm_gather_bytes(nnz, rows, F, weighted, accumulate, mean, empty_rows=0):
    """Algorithmic bytes of one SpMM under the gather model (no cache credit), int32 columns:
    per edge 4F (dense row) + 4 (col) + 4 (val, if weighted); per row 8 (rowptr); per row that is
    written 4F, + 4F when accumulating onto a previous out, + 4 for the mean divisor.  In
    accumulate mode a row without edges is not touched (the reference skips it, spmm.cpp:486; with
    the mean divisor its degree is clamped to 1 and x / 1 == x), so ``empty_rows`` of the ``rows``
    do not count there."""
    per_edge = 4 * F + 4 + (4 if weighted else 0)
    touched = rows - (empty_rows if accumulate else 0)
    per_touched = 4 * F + (4 * F if accumulate else 0) + (4 if mean else 0)
    return nnz * per_edge + rows * 8 + touched * per_touched


def quant_bytes(rows, F, bits):
    """Fused quantize+pack (and, read the other way, unpack+dequantize): per row 4F + F*bits/8 + 8."""
    return rows * (4 * F + F * bits // 8 + 8)


def time_steps(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def time_reps_events(fn, reps, warmup, flush=None):
    """Per-repetition device times (ms) from event pairs on the current stream; ``flush`` (a
    callable that overwrites a buffer larger than L2 + Infinity Cache) runs before each repetition,
    outside the timed pair."""
    import torch
    for _ in range(warmup):
        fn()
    times = []
    for _ in range(reps):
        if flush is not None:
            flush()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b))
    times.sort()
    return {"median_ms": round(times[len(times) // 2], 4), "min_ms": round(times[0], 4)}


def build_headline_graph(nodes, und_edges, F, device):
    import torch
    from super_gnn_amd import synth
    t0 = time.perf_counter()
    rowptr, col = synth.rmat_graph(nodes, und_edges, a=0.57, b=0.19, c=0.19, seed=1, device=device)
    w = synth.gcn_norm_weights(rowptr, col)
    g = torch.Generator(device=device)
    g.manual_seed(2)
    x = torch.randn(nodes, F, generator=g, device=device, dtype=torch.float32)
    torch.cuda.synchronize()
    log(f"[bench] graph: {nodes} nodes, {col.numel()} stored edges, max degree "
        f"{int((rowptr[1:] - rowptr[:-1]).max())}, built in {time.perf_counter() - t0:.1f}s")
    deg = rowptr[1:] - rowptr[:-1]
    edges = [0, 1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1 << 30]
    hist = []
    for lo, hi in zip(edges[:-1], edges[1:]):
        m = (deg >= lo) & (deg < hi)
        hist.append(f"[{lo},{hi if hi < (1 << 30) else 'inf'}): {int(m.sum())} rows / {int(deg[m].sum())} edges")
    log("[bench] degree histogram: " + "; ".join(hist))
    return rowptr, col, w, x


def cpu_baseline_spmm(rowptr, col, w, x, target_edges=1 << 40, reps=10):
    """Time the CPU path on the same graph (all rows unless target_edges bounds the sample to the
    leading rows holding that many edges), gathering from the full X.  Uses the reference's own x86
    extension when oracle/_ref is loadable on this host, else the C restatement."""
    import numpy as np
    import torch
    from oracle import oracle as orc
    rp = rowptr.cpu()
    m = int(torch.searchsorted(rp, torch.tensor(target_edges)).item())
    m = max(1, min(m, rp.numel() - 1))
    nnz = int(rp[m])
    rp_s = rp[: m + 1].contiguous()
    col_s = col[:nnz].to(torch.int64).cpu().contiguous()
    w_s = w[:nnz].cpu().contiguous()
    xh = x.cpu()
    F = xh.shape[1]
    out = torch.zeros(m, F)
    ref = orc.ref_ops()
    if ref is not None:
        kind, T = "reference", torch.get_num_threads()
        tgt = torch.linspace(0, nnz, T + 1).to(torch.int64)
        rs = torch.searchsorted(rp_s, tgt).to(torch.int32)  # nnz-balanced contiguous row split
        rs[0], rs[-1] = 0, m
        cs = torch.tensor([0, F], dtype=torch.int32)
        run = lambda: ref.spmm(rp_s, col_s, w_s, xh, out, m, rs, cs)  # noqa: E731
    else:
        kind, T = "port", orc.num_threads()
        a = (rp_s.numpy(), col_s.numpy(), w_s.numpy(), xh.numpy(), out.numpy())
        run = lambda: orc.spmm_accumulate(*a)  # noqa: E731
    run()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        run()
        ts.append(time.perf_counter() - t0)
    t = float(np.median(ts))
    return {"value": nnz / t / 1e9, "unit": "GEdges/s", "cores": int(T), "kind": kind,
            "sample": f"{m} of {rp.numel() - 1} rows ({nnz} edges) of the same graph, full X, F={F}, 1 warm-up + median of {reps}",
            "ms": t * 1e3}


def cpu_baseline_quant(x, bits, rows=200_000, reps=3):
    import numpy as np
    from oracle import oracle as orc
    xs = x[:rows].cpu().numpy()
    orc.quant_rows(xs, [0, rows], bits)
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        orc.quant_rows(xs, [0, rows], bits)
        ts.append(time.perf_counter() - t0)
    t = float(np.median(ts))
    return {"value": quant_bytes(rows, xs.shape[1], bits) / t / 1e9, "unit": "GB/s", "cores": orc.num_threads(),
            "kind": "port", "sample": f"first {rows} rows, int{bits}, median of {reps}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--uniform-rows", type=int, default=0, help="diagnostic: replace the R-MAT graph by uniform random "
                    "rows of --uniform-degree neighbours over --nodes columns")
    ap.add_argument("--uniform-degree", type=int, default=25)
    ap.add_argument("--workload", default="rmat", choices=["rmat", "quant", "copy", "prepost", "sbm", "aggregate", "sage", "small"],
                    help="rmat: headline SpMM (default); quant: int2 quantize+pack as the step; copy: streaming copy; "
                         "prepost: one partition with packed remote rows, fused vs separate; sbm: dense-degree graph, F=602")
    ap.add_argument("--local-nodes", type=int, default=8_000_000)
    ap.add_argument("--remote-nodes", type=int, default=2_000_000)
    ap.add_argument("--local-und-edges", type=int, default=160_000_000)
    ap.add_argument("--remote-edges", type=int, default=80_000_000)
    ap.add_argument("--sbm-nodes", type=int, default=233_000)
    ap.add_argument("--hidden", type=int, default=256, help="sage: hidden width")
    ap.add_argument("--classes", type=int, default=47, help="sage: output classes")
    ap.add_argument("--parts", type=int, default=8, help="aggregate: number of vertex partitions simulated in this process")
    ap.add_argument("--exchange-bits", type=int, default=2, help="aggregate: 32 (fp32 rows) or 8/4/2 (packed)")
    ap.add_argument("--pre", type=int, default=1, help="aggregate: 1 = pre/post aggregation, 0 = plain boundary exchange")
    ap.add_argument("--nodes", type=int, default=2_450_000)
    ap.add_argument("--und-edges", type=int, default=31_000_000)
    ap.add_argument("--feat", type=int, default=128)
    ap.add_argument("--quant-rows", type=int, default=1_000_000)
    ap.add_argument("--quant-feat", type=int, default=256)
    ap.add_argument("--bits", type=int, default=2)
    ap.add_argument("--long-threshold", type=int, default=0, help="SpMM plan: rows longer than this are split (0 = default)")
    ap.add_argument("--piece-edges", type=int, default=0, help="SpMM plan: minimum edges per long-row piece (0 = default)")
    ap.add_argument("--no-extras", action="store_true", help="skip the extra kernels (used under rocprofv3)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this build runs one partition on ONE GPU; there is no multi-GPU path to time "
            f"(--gpus {args.gpus} refused).")
        sys.exit(2)

    import torch
    import super_gnn_amd  # noqa: F401  (raises if libsgnn_hip.so is missing)
    from super_gnn_amd import _lib, synth, supergnn_ops as ops
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    stream = ops._stream

    extra = {}
    # ---- streaming copy yardstick --------------------------------------------------------------
    n_copy = 256 * 1024 * 1024  # 1 GiB in + 1 GiB out
    src = torch.empty(n_copy, device=dev).normal_()
    dst = torch.empty_like(src)
    copy_fn = lambda: _lib.check(_lib.lib.sgnn_stream_copy_f32(src.data_ptr(), dst.data_ptr(), n_copy, stream()))  # noqa: E731
    if args.workload == "copy" or not args.no_extras:
        ms = time_steps(copy_fn, 10, 3)
        extra["stream_copy_GBps"] = round(2 * 4 * n_copy / ms / 1e6, 1)
        log(f"[bench] stream copy: {extra['stream_copy_GBps']} GB/s (read+write)")

    result = None
    if args.workload == "copy":
        _lib.profile_start()
        ms = time_steps(copy_fn, args.steps, args.warmup)
        prof = _lib.profile_stop()
        n, tot = prof["stream_copy_kernel"]
        ach = 2 * 4 * n_copy / (tot / n) / 1e6
        result = {"metric": "stream copy GB/s", "value": round(2 * 4 * n_copy / ms / 1e6, 2), "unit": "GB/s",
                  "config": {"workload": "stream_copy_1GiB"}, "ms_per_step": ms, "dtype": "f32",
                  "roofline": {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                               "frac": round(ach / HBM_PEAK_GBPS, 4), "traffic": None, "kernel": "stream_copy_kernel"},
                  "cpu_baseline": None}
    del src, dst

    # ---- quantize / dequantize sweep -----------------------------------------------------------
    if args.workload == "quant" or not args.no_extras:
        n, F = args.quant_rows, args.quant_feat
        xq = synth.boundary_features(n, F, seed=5, device=dev)
        seg = torch.tensor([0, n], dtype=torch.int32)
        d = torch.empty(n, F, device=dev)
        for bits in (8, 4, 2):
            if args.workload == "quant" and args.no_extras and bits != args.bits:
                continue
            epb = 8 // bits
            q = torch.empty((n + epb - 1) // epb, F, dtype=torch.uint8, device=dev)
            p = torch.empty(n, 2, device=dev)
            qf = lambda: ops.quantize_tensor_for_all_procs(xq, q, p, seg, 1, bits)  # noqa: E731
            df = lambda: ops.dequantize_tensor_for_all_procs(q, d, p, seg, 1, bits)  # noqa: E731
            is_main = args.workload == "quant" and bits == args.bits
            st, wu = (args.steps, args.warmup) if is_main else (10, 3)
            _lib.profile_start()
            ms_q = time_steps(qf, st, wu)
            prof = _lib.profile_stop()
            ms_d = time_steps(df, 10, 3)
            b = quant_bytes(n, F, bits)
            extra[f"quant_pack_int{bits}_GBps"] = round(b / ms_q / 1e6, 1)
            extra[f"unpack_dequant_int{bits}_GBps"] = round(b / ms_d / 1e6, 1)
            log(f"[bench] int{bits}: quantize+pack {b / ms_q / 1e6:.0f} GB/s ({ms_q:.3f} ms), "
                f"unpack+dequant {b / ms_d / 1e6:.0f} GB/s ({ms_d:.3f} ms)")
            if is_main:
                nl, tot = prof["quant_pack_rows_kernel"]
                ach = b / (tot / nl) / 1e6
                wl = f"quant_pack_int{bits}_{n}x{F}"
                result = {"metric": f"quantize-pack GB/s at int{bits}", "value": round(b / ms_q / 1e6, 2),
                          "unit": "GB/s", "config": {"workload": wl, "rows": n, "F": F, "bits": bits},
                          "ms_per_step": ms_q, "dtype": "f32->u8",
                          "roofline": {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBPS,
                                       "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBPS, 4),
                                       "traffic": MEASURED_TRAFFIC_BYTES.get(wl), "kernel": "quant_pack_rows_kernel",
                                       "kernel_avg_ms": round(tot / nl, 5), "algorithmic_bytes": b},
                          "cpu_baseline": None if args.no_cpu else cpu_baseline_quant(xq, bits)}
        if not args.no_cpu and args.workload != "quant":
            extra["cpu_quant_pack_int2"] = cpu_baseline_quant(xq, 2)
        del xq, d

    # ---- headline SpMM -------------------------------------------------------------------------
    if args.workload == "rmat":
        F = args.feat
        if args.uniform_rows:
            g = torch.Generator(device=dev); g.manual_seed(11)
            M, dg = args.uniform_rows, args.uniform_degree
            col = torch.sort(torch.randint(0, args.nodes, (M, dg), generator=g, device=dev), dim=1).values
            col = col.reshape(-1).to(torch.int32).contiguous()
            rowptr = torch.arange(M + 1, device=dev, dtype=torch.int64) * dg
            w = torch.rand(col.numel(), generator=g, device=dev)
            x = torch.randn(args.nodes, F, generator=g, device=dev)
        else:
            rowptr, col, w, x = build_headline_graph(args.nodes, args.und_edges, F, dev)
        M, nnz = rowptr.numel() - 1, col.numel()
        t0 = time.perf_counter()
        plan = ops.SpmmPlan(rowptr, col, x.shape[0], long_row_threshold=args.long_threshold, piece_edges=args.piece_edges)
        torch.cuda.synchronize()
        info = plan.info()
        extra["plan_build_ms"] = round((time.perf_counter() - t0) * 1e3, 1)
        extra["plan"] = {k: info[k] for k in ("long_rows", "pieces", "long_edges", "long_row_threshold", "piece_edges", "partitioned")}
        log(f"[bench] plan: {extra['plan']} built in {extra['plan_build_ms']} ms")
        out = torch.zeros(M, F, device=dev)
        step = lambda: plan.run(w, x, out, accumulate=True)  # noqa: E731
        _lib.profile_start()
        ms = time_steps(step, args.steps, args.warmup)
        prof = _lib.profile_stop()
        per_kernel = {k: round(v[1] / v[0], 5) for k, v in prof.items()}
        log(f"[bench] weighted sum: {ms:.3f} ms/step, {nnz / ms / 1e6:.2f} GEdges/s, kernels (avg ms) {per_kernel}")
        # dominant kernel: the short-row kernel; its share of the algorithmic bytes
        short_edges = nnz - info["long_edges"]
        short_rows = M - info["long_rows"]
        n_empty = int(((rowptr[1:] - rowptr[:-1]) == 0).sum())
        b_short = spmm_gather_bytes(short_edges, short_rows, F, weighted=True, accumulate=True, mean=False, empty_rows=n_empty)
        b_total = spmm_gather_bytes(nnz, M, F, weighted=True, accumulate=True, mean=False, empty_rows=n_empty)
        extra["empty_rows"] = n_empty
        dom = max(prof, key=lambda k: prof[k][1])
        dom_ms = prof[dom][1] / prof[dom][0]
        if dom == "spmm_short_kernel":
            dom_bytes = b_short
        elif dom == "spmm_piece_kernel":
            # per edge: dense row + col + val (the per-unit figure of the gather model); the kernel's own
            # bookkeeping (edge permutation, piece partial sums) is overhead, not algorithmic traffic
            dom_bytes = info["long_edges"] * (4 * F + 8)
        else:
            dom_bytes = b_total
        ach = dom_bytes / dom_ms / 1e6
        wl = f"rmat_{M}n_{nnz}e_F{F}_gcn_weighted_sum" if not args.uniform_rows else f"uniform_{M}x{args.nodes}_deg{args.uniform_degree}_F{F}"
        # mean aggregation (unit weights + fused /deg) as an extra
        if not args.no_extras:
            deg = (rowptr[1:] - rowptr[:-1]).clamp(min=1).to(torch.float32)
            out2 = torch.zeros(M, F, device=dev)
            ms_mean = time_steps(lambda: plan.run(None, x, out2, accumulate=True, row_div=deg), 10, 3)
            extra["spmm_mean_GEdges_per_s"] = round(nnz / ms_mean / 1e6, 3)
            extra["spmm_mean_gather_GBps"] = round(spmm_gather_bytes(nnz, M, F, False, True, True, empty_rows=n_empty) / ms_mean / 1e6, 1)
            del out2
        if not args.no_extras:
            scratch = torch.empty(192 * 1024 * 1024, device=dev)   # 768 MB > 8 x 4 MB L2 + 256 MB Infinity Cache
            extra["spmm_warm"] = time_reps_events(step, 20, 5)
            extra["spmm_cache_flushed"] = time_reps_events(step, 20, 2, flush=lambda: scratch.fill_(1.0))
            log(f"[bench] weighted sum per repetition: warm {extra['spmm_warm']}, caches flushed before each {extra['spmm_cache_flushed']}")
            del scratch
        # one-time preparation, like the plan itself: the unchanged weight tensor was bound during warm-up
        extra["edge_values_bound_to_plan"] = plan._bound is not None
        extra["spmm_total_gather_GBps"] = round(b_total / ms / 1e6, 1)
        extra["spmm_total_frac_of_hbm_peak"] = round(b_total / ms / 1e6 / HBM_PEAK_GBPS, 4)
        extra["spmm_GFLOPs"] = round(2.0 * nnz * F / ms / 1e6, 1)
        extra["kernel_avg_ms"] = per_kernel
        result = {"metric": "SpMM GEdges/s + % HBM roofline (F=128 fp32); quantize-pack GB/s at int2",
                  "value": round(nnz / ms / 1e6, 4), "unit": "GEdges/s",
                  "config": {"workload": wl, "nodes": M, "edges": nnz, "F": F, "aggregation": "weighted_sum",
                             "accumulate": True, "index_dtype": "int32"},
                  "ms_per_step": ms, "dtype": "f32",
                  "roofline": {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                               "frac": round(ach / HBM_PEAK_GBPS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(wl),
                               "kernel": dom, "kernel_avg_ms": round(dom_ms, 5), "algorithmic_bytes": int(dom_bytes)},
                  "cpu_baseline": None if args.no_cpu else cpu_baseline_spmm(rowptr, col, w, x)}

    # ---- the small CPU-runnable configuration: cache-resident, so GEdges/s only -----------------
    if args.workload == "small":
        N, F = 10_000, 128
        g = torch.Generator().manual_seed(0)
        col = torch.randint(0, N, (N, 16), generator=g)
        col = torch.sort(torch.cat([col, torch.arange(N).unsqueeze(1)], dim=1), dim=1).values.reshape(-1)
        rowptr = 17 * torch.arange(N + 1, dtype=torch.int64)
        x = torch.randn(N, F, generator=g)
        w = torch.ones(col.numel())
        d_rowptr, d_col, d_w, d_x = rowptr.to(dev), col.to(torch.int32).to(dev), w.to(dev), x.to(dev)
        plan = ops.SpmmPlan(d_rowptr, d_col, N)
        out = torch.zeros(N, F, device=dev)
        step = lambda: plan.run(d_w, d_x, out, accumulate=True)  # noqa: E731
        _lib.profile_start()
        ms = time_steps(step, args.steps, args.warmup)
        prof = _lib.profile_stop()
        k_ms = prof["spmm_short_kernel"][1] / prof["spmm_short_kernel"][0]
        nnz = col.numel()
        b = spmm_gather_bytes(nnz, N, F, weighted=True, accumulate=True, mean=False)
        xq = torch.randn(2000, F, generator=g).to(dev)
        q = torch.empty(2000, F, dtype=torch.uint8, device=dev); pq = torch.empty(2000, 2, device=dev)
        seg1 = torch.tensor([0, 2000], dtype=torch.int32)
        ms_q = time_steps(lambda: ops.quantize_tensor_for_all_procs(xq, q, pq, seg1, 1, 8), 50, 10)
        cpu = None
        if not args.no_cpu:
            cpu = cpu_baseline_spmm(rowptr, col, w, x, reps=20)
            nt = torch.get_num_threads()
            torch.set_num_threads(1); os.environ["OMP_NUM_THREADS"] = "1"
            cpu1 = cpu_baseline_spmm(rowptr, col, w, x, reps=5)
            torch.set_num_threads(nt)
            extra["cpu_1_thread_GEdges_per_s"] = round(cpu1["value"], 4)
        extra.update({"kernel_ms": round(k_ms, 5), "kernel_GEdges_per_s": round(nnz / k_ms / 1e6, 2),
                      "kernel_gather_GBps_cache_resident": round(b / k_ms / 1e6, 1),
                      "quant_int8_2000x128_us_per_call": round(ms_q * 1e3, 2)})
        log(f"[bench] small: {ms * 1e3:.1f} us/step wall, kernel {k_ms * 1e3:.1f} us = {nnz / k_ms / 1e6:.1f} GEdges/s; int8 quantize 2000x128 {ms_q * 1e3:.1f} us/call")
        result = {"metric": "SpMM GEdges/s (10k nodes x 17 edges, F=128, cache-resident)", "value": round(nnz / ms / 1e6, 4),
                  "unit": "GEdges/s", "config": {"workload": f"small_uniform_{N}n_{nnz}e_F{F}_sum"}, "ms_per_step": ms,
                  "dtype": "f32", "roofline": None, "cpu_baseline": cpu}

    # ---- one partition in pre/post-aggregation mode: remote rows arrive int2-packed -------------
    if args.workload == "prepost":
        F, bits = args.feat, args.bits
        Ml, Kr = args.local_nodes, args.remote_nodes
        t0 = time.perf_counter()
        rp_l, col_l = synth.rmat_graph(Ml, args.local_und_edges, seed=6, device=dev)
        g = torch.Generator(device=dev); g.manual_seed(7)
        # remote edges: rows follow the local degree distribution, columns uniform over the boundary set
        deg_l = (rp_l[1:] - rp_l[:-1]).to(torch.float32)
        rows_r = torch.multinomial(deg_l + 0.05, args.remote_edges, replacement=True, generator=g)
        cols_r = torch.randint(0, Kr, (args.remote_edges,), generator=g, device=dev)
        rp_r, col_r = synth.csr_from_pairs(rows_r, cols_r, Ml, Kr, dedupe=True)
        del rows_r, cols_r, deg_l
        x_l = torch.randn(Ml, F, generator=g, device=dev)
        x_r = torch.randn(Kr, F, generator=g, device=dev)
        torch.cuda.synchronize()
        log(f"[bench] prepost: local {Ml} rows / {col_l.numel()} edges, remote {Kr} cols / {col_r.numel()} edges, "
            f"built in {time.perf_counter() - t0:.1f}s")
        P = 8
        wr = torch.tensor([Kr * i // P for i in range(P + 1)], dtype=torch.int32)
        epb = 8 // bits
        npk = sum((int(wr[i + 1] - wr[i]) + epb - 1) // epb for i in range(P))
        q = torch.empty(npk, F, dtype=torch.uint8, device=dev)
        prm = torch.empty(Kr, 2, device=dev)
        ops.quantize_tensor_for_all_procs(x_r, q, prm, wr, P, bits)
        del x_r
        plan_l = ops.SpmmPlan(rp_l, col_l, Ml)
        plan_r = ops.SpmmPlan(rp_r, col_r, Kr)
        segs = ops.quant_segments(wr, bits)
        out = torch.zeros(Ml, F, device=dev)
        recv = torch.empty(Kr, F, device=dev)
        ms_local = time_steps(lambda: plan_l.run(None, x_l, out, accumulate=True), args.steps, args.warmup)

        def separate():
            ops.dequantize_tensor_for_all_procs(q, recv, prm, wr, P, bits)
            plan_r.run(None, recv, out, accumulate=True)

        ms_sep = time_steps(separate, args.steps, args.warmup)
        _lib.profile_start()
        ms_fused = time_steps(lambda: plan_r.run_quantized(None, q, prm, segs, bits, out, accumulate=True), args.steps, args.warmup)
        prof = _lib.profile_stop()
        nl, nr = col_l.numel(), col_r.numel()
        per_kernel = {k: round(v[1] / v[0], 5) for k, v in prof.items()}
        dom = max(prof, key=lambda k: prof[k][1])
        info_r = plan_r.info()
        dom_edges = info_r["long_edges"] if "piece" in dom else nr - info_r["long_edges"]
        dom_bytes = dom_edges * (F + 16)  # survey figure for a remote edge: one packed row of F bytes + params + col/val
        dom_ms = prof[dom][1] / prof[dom][0]
        extra.update({"local_spmm_ms": round(ms_local, 4), "remote_separate_ms": round(ms_sep, 4),
                      "remote_fused_ms": round(ms_fused, 4), "fused_speedup_on_remote_step": round(ms_sep / ms_fused, 3),
                      "local_GEdges_per_s": round(nl / ms_local / 1e6, 3), "kernel_avg_ms": per_kernel})
        log(f"[bench] local SpMM {ms_local:.3f} ms; remote: separate {ms_sep:.3f} ms vs fused {ms_fused:.3f} ms")
        total = ms_local + ms_fused
        result = {"metric": "SpMM GEdges/s, pre/post-aggregation partition (local fp32 + int2-packed remote rows, fused)",
                  "value": round((nl + nr) / total / 1e6, 4), "unit": "GEdges/s",
                  "config": {"workload": f"prepost_{Ml}n_{nl}e_local_{Kr}c_{nr}e_remote_int{bits}_F{F}", "F": F, "bits": bits},
                  "ms_per_step": total, "dtype": "f32",
                  "roofline": {"bound": "hbm", "achieved": round(dom_bytes / dom_ms / 1e6, 1), "peak": HBM_PEAK_GBPS,
                               "unit": "GB/s", "frac": round(dom_bytes / dom_ms / 1e6 / HBM_PEAK_GBPS, 4), "traffic": None,
                               "kernel": dom, "kernel_avg_ms": round(dom_ms, 5), "algorithmic_bytes": int(dom_bytes)},
                  "cpu_baseline": None}

    # ---- dense-degree community graph, wide odd feature rows --------------------------------------
    if args.workload == "sbm":
        F = 602
        n = args.sbm_nodes // 50 * 50
        t0 = time.perf_counter()
        rowptr, col = synth.sbm_graph(n, 50, 0.03048, 0.001524, seed=3, device=dev)
        g = torch.Generator(device=dev); g.manual_seed(4)
        x = torch.rand(n, F, generator=g, device=dev) * 2 - 1
        torch.cuda.synchronize()
        nnz = col.numel()
        log(f"[bench] sbm: {n} nodes, {nnz} edges (avg degree {nnz / n:.0f}), built in {time.perf_counter() - t0:.1f}s")
        plan = ops.SpmmPlan(rowptr, col, n, long_row_threshold=args.long_threshold, piece_edges=args.piece_edges)
        info = plan.info()
        out = torch.zeros(n, F, device=dev)
        _lib.profile_start()
        ms = time_steps(lambda: plan.run(None, x, out, accumulate=True), args.steps, args.warmup)
        prof = _lib.profile_stop()
        per_kernel = {k: round(v[1] / v[0], 5) for k, v in prof.items()}
        dom = max(prof, key=lambda k: prof[k][1])
        dom_ms = prof[dom][1] / prof[dom][0]
        dom_edges = info["long_edges"] if "piece" in dom else nnz - info["long_edges"]
        dom_bytes = dom_edges * (4 * F + 4)
        b_total = spmm_gather_bytes(nnz, n, F, weighted=False, accumulate=True, mean=False,
                                    empty_rows=int(((rowptr[1:] - rowptr[:-1]) == 0).sum()))
        extra.update({"kernel_avg_ms": per_kernel, "plan": {k: info[k] for k in ("long_rows", "pieces", "long_edges")},
                      "spmm_total_gather_GBps": round(b_total / ms / 1e6, 1)})
        log(f"[bench] sbm sum: {ms:.3f} ms/step, {nnz / ms / 1e6:.2f} GEdges/s, {b_total / ms / 1e6:.0f} GB/s gather model, {per_kernel}")
        result = {"metric": "SpMM GEdges/s (dense-degree community graph, F=602 fp32)", "value": round(nnz / ms / 1e6, 4),
                  "unit": "GEdges/s", "config": {"workload": f"sbm_{n}n_{nnz}e_F{F}_sum", "F": F}, "ms_per_step": ms,
                  "dtype": "f32",
                  "roofline": {"bound": "hbm", "achieved": round(dom_bytes / dom_ms / 1e6, 1), "peak": HBM_PEAK_GBPS,
                               "unit": "GB/s", "frac": round(dom_bytes / dom_ms / 1e6 / HBM_PEAK_GBPS, 4), "traffic": None,
                               "kernel": dom, "kernel_avg_ms": round(dom_ms, 5), "algorithmic_bytes": int(dom_bytes)},
                  "cpu_baseline": None}

    # ---- one GraphSAGE-style aggregation (forward + backward) over P partitions of the headline graph ----
    if args.workload == "aggregate":
        from super_gnn_amd.aggregator import LoopbackWorld
        from super_gnn_amd.data_manager import build_loopback_partitions
        F = args.feat
        rowptr, col, w, x = build_headline_graph(args.nodes, args.und_edges, F, dev)
        t0 = time.perf_counter()
        graphs = build_loopback_partitions(rowptr, col, w, args.parts, F, num_bits=args.exchange_bits,
                                           is_pre_delay=bool(args.pre), device=dev)
        log(f"[bench] {args.parts} partitions built in {time.perf_counter() - t0:.1f}s; rows exchanged per direction: "
            f"{sum(sum(g.comm_splits.send_splits) for g in graphs)}")
        world = LoopbackWorld(graphs, args.exchange_bits, bool(args.pre))
        feats = [x[g.node_range[0]:g.node_range[1]].clone().requires_grad_() for g in graphs]
        grads = [torch.randn(g.node_range[1] - g.node_range[0], F, device=dev) for g in graphs]

        def step():
            outs = world.aggregate(feats)
            torch.autograd.backward(outs, grads)
            for f in feats:
                f.grad = None

        ms = time_steps(step, args.steps, args.warmup)
        ms_fwd = time_steps(lambda: world.aggregate([f.detach() for f in feats]), args.steps, args.warmup)
        nnz = col.numel()
        extra.update({"forward_ms": round(ms_fwd, 4), "forward_backward_ms": round(ms, 4),
                      "rows_exchanged": sum(sum(g.comm_splits.send_splits) for g in graphs)})
        log(f"[bench] aggregate fwd {ms_fwd:.3f} ms, fwd+bwd {ms:.3f} ms ({2 * nnz / ms / 1e6:.2f} GEdges/s)")
        result = {"metric": "aggregation layer GEdges/s (forward+backward, loop-back exchange)",
                  "value": round(2 * nnz / ms / 1e6, 4), "unit": "GEdges/s",
                  "config": {"workload": f"aggregate_rmat_{args.nodes}n_{nnz}e_F{F}_P{args.parts}_bits{args.exchange_bits}_pre{args.pre}"},
                  "ms_per_step": ms, "dtype": "f32", "roofline": None, "cpu_baseline": None}

    # ---- one training epoch of a 3-layer GraphSAGE over P partitions (examples/graphsage/sage.py:213-232) ----
    if args.workload == "sage":
        from super_gnn_amd.aggregator import LoopbackWorld
        from super_gnn_amd.data_manager import build_loopback_partitions
        from super_gnn_amd.layers import LoopbackSAGE
        F, H, C = args.feat, args.hidden, args.classes
        rowptr, col, _, x = build_headline_graph(args.nodes, args.und_edges, F, dev)
        graphs = build_loopback_partitions(rowptr, col, None, args.parts, max(F, H, C), num_bits=args.exchange_bits,
                                           is_pre_delay=bool(args.pre), device=dev)
        world = LoopbackWorld(graphs, args.exchange_bits, bool(args.pre),
                              params_wire_dtype=torch.bfloat16 if args.exchange_bits in (2, 4, 8) else None)
        torch.manual_seed(0)
        model = LoopbackSAGE(F, H, C, num_layers=3, dropout=0.5).to(dev)
        model.reset_parameters()
        opt = torch.optim.Adam(model.parameters(), lr=0.01)
        feats = [x[g.node_range[0]:g.node_range[1]] for g in graphs]
        labels = torch.randint(0, C, (rowptr.numel() - 1,), device=dev)

        def epoch():
            model.train()
            opt.zero_grad()
            out = torch.cat(model(world, feats))
            # nll_loss(out, labels) written as a gather: torch's nll_loss kernels reduce 2.45 M rows in a
            # single workgroup (5 ms forward, 4 ms backward)
            loss = -out.gather(1, labels.view(-1, 1)).mean()
            loss.backward()
            opt.step()

        ms = time_steps(epoch, args.steps, args.warmup)
        nnz = col.numel()
        log(f"[bench] sage epoch {ms:.3f} ms (3 layers {F}-{H}-{H}-{C}, P={args.parts}, bits={args.exchange_bits}, pre={args.pre})")
        result = {"metric": "GraphSAGE training epoch time (3 layers, full graph, loop-back exchange)",
                  "value": round(1000.0 / ms, 4), "unit": "epochs/s",
                  "config": {"workload": f"sage_rmat_{args.nodes}n_{nnz}e_F{F}_H{H}_C{C}_P{args.parts}_bits{args.exchange_bits}_pre{args.pre}"},
                  "ms_per_step": ms, "dtype": "f32", "roofline": None, "cpu_baseline": None}

    line = {"metric": result["metric"], "value": result["value"], "unit": result["unit"], "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(result["ms_per_step"], 5),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": result["dtype"],
            "data": "synthetic", "config": result["config"], "roofline": result["roofline"],
            "cpu_baseline": result["cpu_baseline"], "extra": extra}
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
