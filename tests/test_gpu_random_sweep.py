"""Seeded random sweeps over shapes the fixed cases do not list: every configuration is derived from
its index, so a failure names a reproducible case.  Same bars as the fixed tests: SpMM within
rel 1e-5 / abs 1e-6 of the oracle (long rows adjudicated against fp64), quantized bytes and params
bit-exact, dequantized floats within one rounding of code*scale."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from _util import random_csr, abs_sum64, assert_spmm_close, dequant_atol

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", range(40))
def test_spmm_random_shapes(case):
    from super_gnn_amd import supergnn_ops as ops
    rng = np.random.default_rng(1000 + case)
    M, K = int(rng.integers(1, 3000)), int(rng.integers(1, 3000))
    F = int(rng.choice([1, 3, 4, 8, 30, 32, 64, 100, 128, 130, 256, 300, 602, 1028]))
    deg = float(rng.choice([0.3, 1, 4, 17, 60]))
    hubs = int(rng.integers(0, 4)) if M > 8 else 0
    rowptr, col, val = random_csr(M, K, deg, seed=case, empty_frac=float(rng.choice([0, 0.3, 0.9])), hubs=hubs,
                                  hub_deg=int(rng.integers(100, 4000)), dup=bool(rng.integers(0, 2)))
    x = rng.standard_normal((K, F)).astype(np.float32)
    init = rng.standard_normal((M, F)).astype(np.float32)
    accumulate = bool(rng.integers(0, 2))
    weighted = bool(rng.integers(0, 3))           # 1 in 3: unit weights passed as None
    mean = bool(rng.integers(0, 2))
    thresh = int(rng.choice([0, 8, 40, 128]))
    piece = int(rng.choice([0, 8, 32]))
    dev = torch.device("cuda:0")
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev).to(torch.int32 if case % 2 else torch.int64),
                        K, long_row_threshold=thresh, piece_edges=piece)
    div = np.maximum(np.diff(rowptr), 1).astype(np.float32) if mean else None
    v = val if weighted else None
    out = torch.from_numpy(init.copy()).to(dev)
    for _ in range(2 if case % 3 == 0 else 1):    # the second call runs with the values bound to the plan
        out.copy_(torch.from_numpy(init))
        plan.run(torch.from_numpy(v).to(dev) if v is not None else None, torch.from_numpy(x).to(dev), out,
                 accumulate=accumulate, row_div=torch.from_numpy(div).to(dev) if mean else None)
    got = out.cpu().numpy()
    want = init.copy() if accumulate else np.zeros_like(init)
    ones = np.ones(col.shape[0], np.float32)
    (orc.spmm_accumulate if accumulate else orc.spmm_overwrite)(rowptr, col, v if v is not None else ones, x, want)
    base = init if accumulate else None
    f64 = orc.spmm_f64(rowptr, col, v if v is not None else ones, x, base)
    asum = abs_sum64(rowptr, col, v if v is not None else ones, x, base)
    if mean:
        orc.row_divide(want, div)
        f64 = f64 / div[:, None].astype(np.float64)
        asum = asum / div[:, None].astype(np.float64)
    assert_spmm_close(got, want, f64, asum, np.diff(rowptr), what=f"case {case}: M={M} K={K} F={F} deg={deg} acc={accumulate} mean={mean}")


@pytest.mark.parametrize("case", range(40))
def test_quant_random_shapes(case):
    from super_gnn_amd import supergnn_ops as ops
    rng = np.random.default_rng(2000 + case)
    bits = int(rng.choice([8, 4, 2]))
    F = int(rng.choice([1, 2, 4, 7, 16, 64, 100, 128, 255, 256, 600, 1024, 1030, 2050]))
    P = int(rng.choice([1, 1, 2, 5, 16]))
    sizes = rng.integers(0, 200, size=P)
    seg = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    n = int(seg[-1])
    if n == 0:
        seg[-1] = n = 3
    x = (rng.standard_normal((n, F)) * np.exp(rng.uniform(-10, 10, size=(n, 1)))).astype(np.float32)
    x[rng.random(n) < 0.05] = 0.0
    x[rng.random(n) < 0.05] = 1.5              # constant rows: scale 0 -> 1
    q_ref, p_ref = orc.quant_rows(x, seg, bits)
    seg_t = torch.from_numpy(seg)
    bf16 = bool(rng.integers(0, 2))
    q = torch.zeros(q_ref.shape, dtype=torch.uint8, device="cuda")
    prm = torch.zeros((n, 2), device="cuda", dtype=torch.bfloat16 if bf16 else torch.float32)
    xd = torch.from_numpy(x).cuda()
    if case % 4 == 0:                           # through a row index over a larger, strided source
        src = torch.zeros((n + 50, F + 4), device="cuda")
        perm = torch.randperm(n + 50, generator=torch.Generator().manual_seed(case))[:n].cuda()
        src[perm, 2:2 + F] = xd
        ops.quantize_tensor_for_all_procs(src[:, 2:2 + F], q, prm, seg_t, P, bits, row_index=perm)
    else:
        ops.quantize_tensor_for_all_procs(xd, q, prm, seg_t, P, bits)
    assert np.array_equal(q.cpu().numpy(), q_ref), f"case {case}: bits={bits} F={F} P={P} n={n}"
    want_p = torch.from_numpy(p_ref).to(torch.bfloat16) if bf16 else torch.from_numpy(p_ref)
    assert torch.equal(prm.cpu(), want_p)
    back = torch.zeros((n, F), device="cuda")
    ops.dequantize_tensor_for_all_procs(q, back, prm, seg_t, P, bits)
    p_used = prm.to(torch.float32).cpu().numpy()
    want = orc.dequant_rows(q_ref, p_used, seg, bits, F)
    tol = dequant_atol(p_used[:, 0], p_used[:, 1], bits)[:, None]
    assert np.all(np.abs(back.cpu().numpy() - want) <= tol), f"case {case}"


@pytest.mark.parametrize("stream", ["default", "1", "0"])
@pytest.mark.parametrize("case", range(40))
def test_quant_rows_by_index_pitch_and_special_values(case, stream, monkeypatch):
    """Quantizer input rows that are consecutive, picked by a row index (repeats, the source's last row), read with a
    pitch out of a wider tensor, or both; rows with a NaN first / later, infinities, zeros of both signs, constants;
    ragged per-peer segments; output at odd addresses -- under the default choice of kernel and with either
    quantizer family forced (SGNN_QUANT_STREAM).  Bytes and params bit for bit against the oracle on the gathered copy."""
    from super_gnn_amd import supergnn_ops as ops
    if stream != "default":
        monkeypatch.setenv("SGNN_QUANT_STREAM", stream)
    rng = np.random.default_rng(7000 + case)
    F = int(rng.choice([9, 10, 12, 13, 16, 17, 33, 37, 64, 100, 123, 128, 250, 256, 301, 602, 640, 1000, 1026, 1433, 1538, 2050, 2562, 3703, 4100]))
    n = int(rng.integers(1, 2500)) if F < 1100 else int(rng.integers(1, 300))
    bits = int(rng.choice([8, 4, 2]))
    P = int(rng.choice([1, 1, 2, 5, 13, 64, 65]))
    mode = case % 4                             # 0 consecutive, 1 index, 2 pitch, 3 index + pitch
    n_src = n if mode in (0, 2) else int(rng.integers(1, 2 * n + 2))
    pitch = F if mode in (0, 1) else F + int(rng.integers(1, 9))
    col0 = 0 if pitch == F else int(rng.integers(0, pitch - F + 1))
    src = (rng.standard_normal((n_src, pitch)) * np.exp(rng.uniform(-3, 3, size=(n_src, 1)))).astype(np.float32)
    for r in rng.integers(0, n_src, size=max(1, n_src // 7)):
        kind, c = int(rng.integers(0, 6)), col0 + int(rng.integers(0, F))
        row = src[r, col0:col0 + F]
        if kind == 0: row[0] = np.nan
        elif kind == 1: src[r, c] = np.nan
        elif kind == 2: src[r, c] = np.inf if rng.random() < 0.5 else -np.inf
        elif kind == 3: row[:] = np.abs(row); src[r, c] = -0.0 if rng.random() < 0.5 else 0.0; row[int(rng.integers(0, F))] = 0.0
        elif kind == 4: row[:] = np.float32(rng.standard_normal())
        else: row[:] = -np.abs(row); src[r, c] = 0.0; row[int(rng.integers(0, F))] = -0.0
    idx = rng.integers(0, n_src, size=n) if mode in (1, 3) else None
    if idx is not None and n > 2:
        idx[int(rng.integers(0, n))] = n_src - 1
    x = np.ascontiguousarray((src[idx] if idx is not None else src)[:, col0:col0 + F])
    seg = [0] + [int(c) for c in np.sort(rng.integers(0, n + 1, size=P - 1))] + [n]
    q_ref, p_ref = orc.quant_rows(x, seg, bits)
    npk, qoff = q_ref.shape[0], int(rng.integers(0, 4))
    qb = torch.full((npk * F + 8,), 0xCD, dtype=torch.uint8, device="cuda")
    prm = torch.zeros(n, 2, device="cuda")
    ops.quantize_tensor_for_all_procs(torch.from_numpy(src).cuda()[:, col0:col0 + F], qb[qoff:qoff + npk * F].view(npk, F), prm,
                                      torch.tensor(seg, dtype=torch.int32), P, bits,
                                      row_index=None if idx is None else torch.from_numpy(idx).cuda())
    got, pg, nan_ref = qb.cpu().numpy(), prm.cpu().numpy(), np.isnan(p_ref)
    what = f"case {case}: n={n} F={F} bits={bits} P={P} mode={mode} pitch={pitch} col0={col0} qoff={qoff}"
    assert np.array_equal(np.isnan(pg), nan_ref), what
    assert np.array_equal(pg[~nan_ref].view(np.uint32), p_ref[~nan_ref].view(np.uint32)), what
    assert np.array_equal(got[qoff:qoff + npk * F].reshape(npk, F), q_ref), what
    assert (got[:qoff] == 0xCD).all() and (got[qoff + npk * F:] == 0xCD).all(), what + ": bytes outside the rows were written"


@pytest.mark.parametrize("case", range(30))
def test_fused_random_shapes(case):
    # random widths (every lane-group shape), ragged segments, hub rows, fp32 / bf16 params, all epilogues:
    # the fused product must equal dequantize-then-SpMM on the same plan bit for bit
    from super_gnn_amd import supergnn_ops as ops
    rng = np.random.default_rng(3000 + case)
    bits = int(rng.choice([8, 4, 2]))
    F = int(rng.choice([4, 8, 12, 36, 64, 100, 128, 256, 260, 512, 1028, 2, 6, 130, 602, 1030]))
    M, K = int(rng.integers(1, 1500)), int(rng.integers(8, 1500))
    deg = int(rng.choice([1, 3, 9, 40]))
    hubs = int(rng.choice([0, 0, 3]))
    rowptr, col, val = random_csr(M, K, deg, seed=3000 + case, empty_frac=0.2, hubs=hubs, hub_deg=min(2 * K, 700))
    P = int(rng.choice([1, 2, 7]))
    cuts = np.sort(rng.integers(0, K + 1, size=P - 1))
    seg = np.concatenate([[0], cuts, [K]]).astype(np.int32)
    seg_t = torch.from_numpy(seg)
    x = torch.from_numpy((rng.standard_normal((K, F)) * np.exp(rng.uniform(-3, 3, size=(K, 1)))).astype(np.float32)).cuda()
    bf16 = bool(rng.integers(0, 2))
    npk = int(orc.packed_rows(seg, bits).sum())
    q = torch.zeros(npk, F, dtype=torch.uint8, device="cuda")
    prm = torch.zeros(K, 2, device="cuda", dtype=torch.bfloat16 if bf16 else torch.float32)
    ops.quantize_tensor_for_all_procs(x, q, prm, seg_t, P, bits)
    recv = torch.empty(K, F, device="cuda")
    ops.dequantize_tensor_for_all_procs(q, recv, prm, seg_t, P, bits)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).cuda(), torch.from_numpy(col).cuda(), K,
                        long_row_threshold=int(rng.choice([0, 16, 64])))
    segs = ops.quant_segments(seg_t, bits)
    w = torch.from_numpy(val).cuda() if rng.integers(0, 2) else None
    accumulate = bool(rng.integers(0, 2))
    div = torch.from_numpy(np.maximum(np.diff(rowptr), 1).astype(np.float32)).cuda() if rng.integers(0, 2) else None
    init = torch.from_numpy(rng.standard_normal((M, F)).astype(np.float32)).cuda()
    want, got = init.clone(), init.clone()
    for _ in range(2):   # the second call runs with the weights and row slots bound to the plan
        plan.run(w, recv, want, accumulate=accumulate, row_div=div)
        plan.run_quantized(w, q, prm, segs, bits, got, accumulate=accumulate, row_div=div)
    torch.cuda.synchronize()
    assert torch.equal(got, want), f"case {case}: bits={bits} F={F} M={M} K={K} deg={deg} hubs={hubs} P={P} bf16={bf16}"


@pytest.mark.parametrize("case", range(30))
def test_band_schedule_random_shapes(case, monkeypatch):
    # the column-band schedule forced onto random matrices with random band widths: column-sorted rows must come
    # out bit-identical to the oracle's CSR-order fma chain in every mode
    from super_gnn_amd import supergnn_ops as ops
    rng = np.random.default_rng(4000 + case)
    M, K = int(rng.integers(1, 2000)), int(rng.integers(1, 2500))
    F = int(rng.choice([1, 2, 5, 16, 48, 64, 100, 128, 200, 256, 301, 602, 640, 1030]))
    deg = float(rng.choice([0.5, 3, 12, 50]))
    hubs = int(rng.integers(0, 3)) if M > 8 else 0
    cols = int(rng.choice([1, 7, 32, 100, 256, 1000, 4096]))
    monkeypatch.setenv("SGNN_SPMM_BAND", "1")
    monkeypatch.setenv("SGNN_SPMM_BAND_COLS", str(cols))
    if case % 5 == 0:
        monkeypatch.setenv("SGNN_SPMM_BAND_CHUNK_EDGES", str(int(rng.choice([8, 24, 64]))))
    unsorted = case % 6 == 5                                  # rows in random column order: the schedule must step aside
    rowptr, col, val = random_csr(M, K, deg, seed=4000 + case, empty_frac=float(rng.choice([0, 0.3, 0.9])), hubs=hubs,
                                  hub_deg=int(rng.integers(100, 3000)), dup=unsorted)
    x = rng.standard_normal((K, F)).astype(np.float32)
    init = rng.standard_normal((M, F)).astype(np.float32)
    accumulate, mean, weighted = bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 3))
    dev = torch.device("cuda:0")
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    assert plan.schedule(F)["band"] == int(col.size > 0), "forced on for every matrix that has edges"
    div = np.maximum(np.diff(rowptr), 1).astype(np.float32) if mean else None
    v = val if weighted else np.ones(col.shape[0], np.float32)
    xd = torch.from_numpy(x).to(dev)
    out = torch.from_numpy(init.copy()).to(dev)
    for _ in range(2 if case % 3 == 0 else 1):
        out.copy_(torch.from_numpy(init))
        plan.run(torch.from_numpy(val).to(dev) if weighted else None, xd, out, accumulate=accumulate,
                 row_div=torch.from_numpy(div).to(dev) if mean else None)
    want = init.copy() if accumulate else np.zeros_like(init)
    orc.spmm_accumulate(rowptr, col, v, x, want)
    if mean:
        orc.row_divide(want, div)
    what = f"case {case}: M={M} K={K} F={F} cols={cols} acc={accumulate} mean={mean}"
    if not unsorted:
        assert np.array_equal(out.cpu().numpy(), want), what
        return
    is_sorted = bool(np.all((np.diff(col) >= 0) | np.isin(np.arange(1, col.size), rowptr[1:-1]))) if col.size > 1 else True
    assert plan.schedule(F)["band"] == int(is_sorted and col.size > 0), "known after the first product"
    base = init if accumulate else None
    f64, asum = orc.spmm_f64(rowptr, col, v, x, base), abs_sum64(rowptr, col, v, x, base)
    if mean:
        f64, asum = f64 / div[:, None].astype(np.float64), asum / div[:, None].astype(np.float64)
    assert_spmm_close(out.cpu().numpy(), want, f64, asum, np.diff(rowptr), what=what)
