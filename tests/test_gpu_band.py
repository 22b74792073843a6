"""The band schedule of the SpMM (column bands x feature slices per XCD, one launch per band) against
the CPU oracle.  It sums every row's edges in CSR order with one fma per edge starting from the old
out value, so with column-sorted rows the result must equal the reference's BIT FOR BIT for every row
length -- stronger than the rel 1e-5 / abs 1e-6 bar.  The schedule is forced here (it is normally
chosen only for dense-degree matrices that do not fit the caches) with small bands, so that many bands,
ragged last bands and empty (row, band) pairs occur at sizes the oracle finishes in a blink."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from _util import random_csr, abs_sum64, assert_spmm_close

pytestmark = pytest.mark.gpu


def _ops():
    import super_gnn_amd  # noqa: F401
    from super_gnn_amd import supergnn_ops
    return supergnn_ops


def _force(monkeypatch, cols):
    monkeypatch.setenv("SGNN_SPMM_BAND", "1")
    monkeypatch.setenv("SGNN_SPMM_BAND_COLS", str(cols))


@pytest.mark.parametrize("M,K,F,deg,cols,window", [
    (700, 900, 602, 40, 128, None),    # a window of 512 columns (8 slices of 64 floats) + one of 90 (2 slices of 48: groups of 12 lanes)
    (700, 900, 602, 40, 128, 0),       # the same in one piece: float2 lanes, 8 slices of 38 vectors, 8 bands
    (500, 1000, 128, 30, 100, None),   # float4, 2 slices x 4 row groups; band width not a power of two
    (300, 800, 256, 25, 256, None),    # 4 slices x 2 row groups
    (257, 600, 64, 20, 64, None),      # one slice, 8 row groups
    (300, 500, 123, 20, 70, None),     # scalar lanes
    (200, 400, 100, 15, 50, None),     # float4 with a ragged last slice
    (150, 300, 2052, 9, 40, 0),        # in one piece: slices wider than one register tile
    (150, 300, 2052, 9, 40, None),     # four windows and a remainder of one float4
    (90, 200, 4, 6, 16, None), (90, 200, 1, 6, 16, None), (64, 100, 10, 5, 7, None),
    (400, 5000, 602, 12, 37, None),    # 136 bands, most (row, band) pairs empty
    (300, 700, 768, 25, 90, None),     # 512 + 256: the second window is 4 slices x 2 row groups
    (260, 600, 1024, 20, 64, None),    # two full windows
    (200, 500, 514, 15, 50, None),     # remainder of two floats
    (240, 520, 542, 17, 60, None),     # remainder of 30 columns: one slice, groups of 8 lanes
    (230, 510, 580, 17, 60, None),     # remainder of 68 columns: 2 slices of 36 (groups of 12 lanes)
    (200, 500, 513, 15, 50, None),     # odd width: scalar lanes in both windows
    (200, 500, 1100, 15, 50, None),    # 512 + 512 + 76
    (220, 450, 330, 18, 45, 128),      # windows of 128 columns: 128 + 128 + 74
])
def test_band_schedule_bit_identical_to_oracle(M, K, F, deg, cols, window, monkeypatch):
    ops = _ops()
    _force(monkeypatch, cols)
    if window is not None:
        monkeypatch.setenv("SGNN_SPMM_BAND_WINDOW", str(window))
    rowptr, col, val = random_csr(M, K, deg, seed=M + F, empty_frac=0.1, hubs=3, hub_deg=min(K, 700))
    rng = np.random.default_rng(F)
    x = rng.standard_normal((K, F), dtype=np.float32)
    init = rng.standard_normal((M, F), dtype=np.float32)
    dev = torch.device("cuda:0")
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    sch = plan.schedule(F)
    assert sch["band"] == 1 and sch["band_cols"] == cols and sch["n_bands"] == -(-K // cols)
    w, xd = torch.from_numpy(val).to(dev), torch.from_numpy(x).to(dev)
    deg_f = np.maximum(np.diff(rowptr), 1).astype(np.float32)
    div = torch.from_numpy(deg_f).to(dev)

    want = init.copy(); orc.spmm_accumulate(rowptr, col, val, x, want)
    out = torch.from_numpy(init.copy()).to(dev)
    plan.run(w, xd, out, accumulate=True)
    assert np.array_equal(out.cpu().numpy(), want), "accumulate"
    out2 = torch.from_numpy(init.copy()).to(dev)
    plan.run(w, xd, out2, accumulate=True)     # second call: the weights are bound to the plan now
    assert torch.equal(out, out2)

    # overwrite + mean: (A x) / deg for every row, rows without edges zero
    want0 = np.zeros_like(init); orc.spmm_accumulate(rowptr, col, val, x, want0)
    orc.row_divide(want0, deg_f)
    out3 = torch.from_numpy(init.copy()).to(dev)
    plan.run(w, xd, out3, accumulate=False, row_div=div)
    assert np.array_equal(out3.cpu().numpy(), want0), "overwrite + mean"

    # unit weights (val == NULL), accumulate + mean: (old + A x) / deg, also for rows without edges
    ones = np.ones_like(val)
    want1 = init.copy(); orc.spmm_accumulate(rowptr, col, ones, x, want1)
    orc.row_divide(want1, deg_f)
    out4 = torch.from_numpy(init.copy()).to(dev)
    plan.run(None, xd, out4, accumulate=True, row_div=div)
    assert np.array_equal(out4.cpu().numpy(), want1), "unit weights + mean"


@pytest.mark.parametrize("F", [602, 128, 37])
def test_band_schedule_with_64_bit_gather_offsets(F, monkeypatch):
    # operands of 4 GB and more per feature slice take a kernel variant with 64-bit row offsets; forced here
    ops = _ops()
    _force(monkeypatch, 96)
    monkeypatch.setenv("SGNN_SPMM_BAND_OFF64", "1")
    M, K = 333, 777
    rowptr, col, val = random_csr(M, K, 30, seed=F, empty_frac=0.1, hubs=2, hub_deg=500)
    rng = np.random.default_rng(F)
    x = rng.standard_normal((K, F), dtype=np.float32)
    init = rng.standard_normal((M, F), dtype=np.float32)
    dev = torch.device("cuda:0")
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    want = init.copy(); orc.spmm_accumulate(rowptr, col, val, x, want)
    out = torch.from_numpy(init.copy()).to(dev)
    plan.run(torch.from_numpy(val).to(dev), torch.from_numpy(x).to(dev), out, accumulate=True)
    assert np.array_equal(out.cpu().numpy(), want)


def test_band_schedule_row_with_more_than_65535_edges_in_one_band(monkeypatch):
    # a chunk's row offsets are 16-bit; a row that long is a chunk of its own and takes its bounds from the header
    ops = _ops()
    _force(monkeypatch, 150000)
    M, K, F = 40, 200000, 16
    rng = np.random.default_rng(7)
    deg = rng.integers(0, 30, size=M)
    deg[17] = 120000
    deg[18] = 70000
    rowptr = np.zeros(M + 1, np.int64); np.cumsum(deg, out=rowptr[1:])
    col = np.concatenate([np.sort(rng.choice(K, size=d, replace=False)) for d in deg]).astype(np.int64)
    val = rng.random(col.size, dtype=np.float32)
    x = rng.standard_normal((K, F), dtype=np.float32)
    init = rng.standard_normal((M, F), dtype=np.float32)
    dev = torch.device("cuda:0")
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    assert plan.schedule(F)["n_bands"] == 2
    for v in (val, None):
        want = init.copy(); orc.spmm_accumulate(rowptr, col, v if v is not None else np.ones_like(val), x, want)
        out = torch.from_numpy(init.copy()).to(dev)
        plan.run(torch.from_numpy(v).to(dev) if v is not None else None, torch.from_numpy(x).to(dev), out, accumulate=True)
        assert np.array_equal(out.cpu().numpy(), want), "weighted" if v is not None else "unit weights"


def test_band_schedule_equals_row_class_schedule_and_honours_rebinding(monkeypatch):
    ops = _ops()
    dev = torch.device("cuda:0")
    M, K, F = 3000, 2000, 128
    rowptr, col, val = random_csr(M, K, 60, seed=5, hubs=4, hub_deg=1500)
    x = torch.randn(K, F, generator=torch.Generator().manual_seed(1)).to(dev)
    w = torch.from_numpy(val).to(dev)
    rp, cl = torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev)
    monkeypatch.setenv("SGNN_SPMM_BAND", "0")
    ref = torch.zeros(M, F, device=dev)
    ops.SpmmPlan(rp, cl, K).run(w, x, ref, accumulate=True)
    _force(monkeypatch, 300)
    plan = ops.SpmmPlan(rp, cl, K)
    out = torch.zeros(M, F, device=dev)
    for _ in range(3):                          # 2nd call binds, 3rd reuses the bound copy
        out.zero_()
        plan.run(w, x, out, accumulate=True)
    short = torch.from_numpy(np.diff(rowptr) <= 128).to(dev)
    assert torch.equal(out[short], ref[short])                    # both schedules: reference order on short rows
    xn = x.cpu().numpy()
    want = np.zeros((M, F), np.float32); orc.spmm_accumulate(rowptr, col, val, xn, want)
    assert np.array_equal(out.cpu().numpy(), want)                # the band schedule: reference order on every row
    assert_spmm_close(ref.cpu().numpy(), want, orc.spmm_f64(rowptr, col, val, xn, None), abs_sum64(rowptr, col, val, xn, None),
                      np.diff(rowptr), what="row-class schedule")  # long rows there: other order, same bar
    # in-place edit of the bound weights: the version counter moves, the plan must not use its stale copy
    w.mul_(2.0)
    out2 = torch.zeros(M, F, device=dev)
    plan.run(w, x, out2, accumulate=True)
    assert torch.equal(out2, out * 2.0)
    # another tensor of weights altogether
    w3 = torch.rand_like(w)
    out3 = torch.zeros(M, F, device=dev)
    plan.run(w3, x, out3, accumulate=True)
    want3 = np.zeros((M, F), np.float32)
    orc.spmm_accumulate(rowptr, col, w3.cpu().numpy(), x.cpu().numpy(), want3)
    assert np.array_equal(out3.cpu().numpy(), want3)


def test_unsorted_rows_keep_the_row_class_schedule(monkeypatch):
    ops = _ops()
    _force(monkeypatch, 64)
    dev = torch.device("cuda:0")
    M, K, F = 400, 500, 64
    rowptr, col, val = random_csr(M, K, 30, seed=9, dup=True)    # columns in random order inside each row
    assert any(np.any(np.diff(col[rowptr[r]:rowptr[r + 1]]) < 0) for r in range(M))
    x = np.random.default_rng(2).standard_normal((K, F), dtype=np.float32)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    out = torch.zeros(M, F, device=dev)
    plan.run(torch.from_numpy(val).to(dev), torch.from_numpy(x).to(dev), out, accumulate=True)
    want = np.zeros((M, F), np.float32); orc.spmm_accumulate(rowptr, col, val, x, want)
    assert np.array_equal(out.cpu().numpy(), want)               # all rows short: CSR order either way
    assert plan.schedule(F)["band"] == 0                          # the plan has seen that rows are unsorted


def test_band_schedule_with_leading_dimensions_through_the_c_abi(monkeypatch):
    ops = _ops()
    from super_gnn_amd._lib import lib, check
    _force(monkeypatch, 90)
    dev = torch.device("cuda:0")
    M, K, F = 600, 700, 602
    rowptr, col, val = random_csr(M, K, 35, seed=31, empty_frac=0.05)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    g = torch.Generator().manual_seed(3)
    xw = torch.randn(K, F + 6, generator=g).to(dev)
    ow = torch.randn(M, F + 10, generator=g).to(dev)
    w = torch.from_numpy(val).to(dev)
    got = ow.clone()
    check(lib.sgnn_spmm_csr_f32(plan._h, w.data_ptr(), xw.data_ptr() + 8, got.data_ptr() + 16, F, F + 6, F + 10, 1, None,
                                torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    want = ow[:, 4:4 + F].cpu().numpy().copy()
    orc.spmm_accumulate(rowptr, col, val, xw[:, 2:2 + F].contiguous().cpu().numpy(), want)
    assert np.array_equal(got[:, 4:4 + F].cpu().numpy(), want)
    keep = torch.ones(F + 10, dtype=torch.bool, device=dev); keep[4:4 + F] = False
    assert torch.equal(got[:, keep], ow[:, keep])


def test_full_size_community_graph_takes_the_band_schedule_and_matches_oracle():
    # the dense-degree configuration at full size with real-valued features: 233 k nodes, ~114 M edges, F = 602
    from super_gnn_amd import synth
    ops = _ops()
    dev = torch.device("cuda:0")
    n, F = 233_000, 602
    rowptr, col = synth.sbm_graph(n, 50, 0.03048, 0.001524, seed=3, device=dev)
    g = torch.Generator(device=dev); g.manual_seed(4)
    x = torch.rand(n, F, generator=g, device=dev) * 2 - 1
    plan = ops.SpmmPlan(rowptr, col, n)
    sch = plan.schedule(F)
    print(f"\n[cfg3] schedule {sch}", flush=True)
    assert sch["band"] == 1 and sch["n_bands"] >= 8
    out = torch.zeros(n, F, device=dev)
    plan.run(None, x, out, accumulate=True)
    torch.cuda.synchronize()
    rp, cl = rowptr.cpu().numpy(), col.cpu().numpy().astype(np.int64)
    want = np.zeros((n, F), np.float32)
    orc.spmm_accumulate(rp, cl, np.ones(cl.shape[0], np.float32), x.cpu().numpy(), want)
    assert np.array_equal(out.cpu().numpy(), want), "band schedule: the reference's fma chain, bit for bit"


def test_schedule_is_chosen_from_the_matrix_shape():
    # the plan-time rule: a dense-degree matrix whose operand overflows the caches takes the band schedule, a
    # power-law graph of the same size (few edges per row and band) and a small matrix keep the row-class kernels
    from super_gnn_amd import synth
    ops = _ops()
    dev = torch.device("cuda:0")
    rp, cl = synth.sbm_graph(60000, 10, 0.02, 0.001, seed=3, device=dev)              # ~170 edges per row
    dense = ops.SpmmPlan(rp, cl, 60000)
    assert dense.schedule(602)["band"] == 1 and dense.schedule(602)["n_slices"] == 10   # a window of 8 slices + one of 2
    assert dense.schedule(512)["n_slices"] == 8 and dense.schedule(256)["n_slices"] == 4
    assert dense.schedule(64)["band"] == 0                                             # 15 MB of X: cache-resident
    rp, cl = synth.rmat_graph(200000, 2500000, seed=1, device=dev)                     # 25 edges per row
    power = ops.SpmmPlan(rp, cl, 200000)
    assert power.schedule(602)["band"] == 0 and power.schedule(128)["band"] == 0


def test_band_schedule_replays_from_a_captured_graph(monkeypatch):
    # steady-state products of the band schedule (restage + one launch per band, more than 48 KB of LDS per
    # workgroup) only launch kernels: capture once, replay with eager work in between, compare bits
    ops = _ops()
    _force(monkeypatch, 256)
    dev = torch.device("cuda:0")
    M, K, F = 900, 1500, 602
    rowptr, col, val = random_csr(M, K, 40, seed=21, empty_frac=0.1, hubs=2, hub_deg=900)
    x = torch.randn(K, F, generator=torch.Generator().manual_seed(3)).to(dev)
    w = torch.from_numpy(val).to(dev)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    out, out1 = torch.zeros(M, F, device=dev), torch.zeros(M, F, device=dev)

    def step():
        out.zero_(); out1.zero_()
        plan.run(w, x, out, accumulate=True)
        plan.run(None, x, out1, accumulate=True)

    for _ in range(3):
        step()
    torch.cuda.synchronize()
    want, want1 = out.clone(), out1.clone()
    ref = np.zeros((M, F), np.float32); orc.spmm_accumulate(rowptr, col, val, x.cpu().numpy(), ref)
    assert np.array_equal(want.cpu().numpy(), ref)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for i in range(3):
        out.fill_(float(i)); out1.fill_(-2.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want) and torch.equal(out1, want1), f"replay {i}"
