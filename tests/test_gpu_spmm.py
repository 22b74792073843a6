"""GPU parity of the SpMM path: libsgnn_hip (through the C ABI) against the CPU restatement in
oracle/ on identical seeded inputs.  Tolerance is the one the task states for fp32 SpMM:
|gpu - ref| <= 1e-6 + 1e-5 * |ref| (summation order may differ on long rows); rows no longer than
the long-row threshold are additionally required to be bit-identical, because the kernel performs
the reference's fma sequence in the reference's order."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from oracle import oracle as orc
from _util import random_csr, abs_sum64 as _abs_sum64, assert_spmm_close as _assert_close

pytestmark = pytest.mark.gpu



def _gpu():
    import super_gnn_amd  # noqa: F401
    from super_gnn_amd import supergnn_ops
    return supergnn_ops


def _run_gpu(rowptr, col, val, x, init, accumulate, row_div=None, col_dtype=torch.int64, thresh=0, seg=0):
    ops = _gpu()
    dev = torch.device("cuda:0")
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev).to(col_dtype), x.shape[0],
                        long_row_threshold=thresh, piece_edges=seg)
    out = torch.from_numpy(init.copy()).to(dev)
    plan.run(torch.from_numpy(val).to(dev) if val is not None else None, torch.from_numpy(x).to(dev), out,
             accumulate=accumulate, row_div=torch.from_numpy(row_div).to(dev) if row_div is not None else None)
    torch.cuda.synchronize()
    return out.cpu().numpy(), plan


@pytest.mark.parametrize("M,K,F,deg", [
    (1000, 800, 128, 9),     # the headline width: 32 lanes x float4
    (513, 300, 64, 5),       # 16-lane groups
    (300, 200, 32, 7),       # 8-lane groups
    (257, 100, 256, 11),     # full wavefront per row
    (200, 300, 602, 12),     # float2 lanes, 5 vectors per lane (Reddit width)
    (150, 100, 123, 6),      # scalar lanes (odd width)
    (120, 90, 100, 6),       # float4 with a partly idle group
    (64, 50, 1024, 4),       # 4 float4 per lane
    (40, 30, 2052, 3),       # wider than one register tile: feature axis walked in tiles
    (50, 40, 4, 3), (50, 40, 1, 3), (33, 20, 10, 5),
])
def test_accumulate_matches_oracle(M, K, F, deg):
    rowptr, col, val = random_csr(M, K, deg, seed=M * 7 + F, empty_frac=0.15)
    rng = np.random.default_rng(F)
    x = rng.standard_normal((K, F), dtype=np.float32)
    init = rng.standard_normal((M, F), dtype=np.float32)
    want = init.copy(); orc.spmm_accumulate(rowptr, col, val, x, want)
    got, plan = _run_gpu(rowptr, col, val, x, init, accumulate=True)
    _assert_close(got, want, what=f"F={F}")
    assert plan.info()["long_rows"] == 0
    assert np.array_equal(got, want), "short rows must reproduce the reference's fma sequence bit for bit"
    empty = np.diff(rowptr) == 0
    assert np.array_equal(got[empty], init[empty])  # empty rows untouched (spmm.cpp:486)


@pytest.mark.parametrize("F", [128, 602, 64])
def test_overwrite_mode_matches_oracle(F):
    M, K = 700, 500
    rowptr, col, val = random_csr(M, K, 8, seed=F, empty_frac=0.2)
    rng = np.random.default_rng(F + 1)
    x = rng.standard_normal((K, F), dtype=np.float32)
    junk = rng.standard_normal((M, F), dtype=np.float32)
    want = junk.copy(); orc.spmm_overwrite(rowptr, col, val, x, want)
    got, _ = _run_gpu(rowptr, col, val, x, junk, accumulate=False)
    _assert_close(got, want, what=f"overwrite F={F}")
    assert np.all(got[np.diff(rowptr) == 0] == 0)  # empty rows zeroed (reducer.h:70-74)


@pytest.mark.parametrize("F,thresh,seg", [(128, 64, 96), (128, 512, 512), (602, 100, 128), (64, 32, 40), (123, 50, 64), (256, 16, 16)])
def test_long_rows_segment_path(F, thresh, seg):
    M, K = 600, 3000
    rowptr, col, val = random_csr(M, K, 10, seed=F + thresh, empty_frac=0.1, hubs=9, hub_deg=2500)
    rng = np.random.default_rng(5)
    x = rng.standard_normal((K, F), dtype=np.float32)
    init = rng.standard_normal((M, F), dtype=np.float32)
    want = init.copy(); orc.spmm_accumulate(rowptr, col, val, x, want)
    f64 = orc.spmm_f64(rowptr, col, val, x, init)
    S, deg = _abs_sum64(rowptr, col, val, x, init), np.diff(rowptr)
    got, plan = _run_gpu(rowptr, col, val, x, init, accumulate=True, thresh=thresh, seg=seg)
    info = plan.info()
    assert info["long_rows"] >= 9 and info["pieces"] >= info["long_rows"]
    _assert_close(got, want, f64, S, deg, what=f"long rows F={F}")
    short = np.diff(rowptr) <= thresh
    assert np.array_equal(got[short], want[short])
    # run-to-run reproducible (no atomics)
    got2, _ = _run_gpu(rowptr, col, val, x, init, accumulate=True, thresh=thresh, seg=seg)
    assert np.array_equal(got, got2)
    # overwrite mode on the same matrix
    w2 = init.copy(); orc.spmm_overwrite(rowptr, col, val, x, w2)
    g2, _ = _run_gpu(rowptr, col, val, x, init, accumulate=False, thresh=thresh, seg=seg)
    _assert_close(g2, w2, orc.spmm_f64(rowptr, col, val, x), _abs_sum64(rowptr, col, val, x), deg, what="long rows overwrite")


def test_mean_epilogue_and_unit_weights():
    M, K, F = 900, 700, 128
    rowptr, col, _ = random_csr(M, K, 14, seed=3, empty_frac=0.1, hubs=2, hub_deg=1500)
    rng = np.random.default_rng(9)
    x = rng.standard_normal((K, F), dtype=np.float32)
    deg = np.maximum(np.diff(rowptr), 1).astype(np.float32)
    ones = np.ones(col.shape[0], dtype=np.float32)
    want = np.zeros((M, F), np.float32); orc.spmm_accumulate(rowptr, col, ones, x, want); orc.row_divide(want, deg)
    f64 = orc.spmm_f64(rowptr, col, ones, x) / deg[:, None]
    S, dg = _abs_sum64(rowptr, col, ones, x) / deg[:, None], np.diff(rowptr)
    got, _ = _run_gpu(rowptr, col, None, x, np.zeros((M, F), np.float32), accumulate=True, row_div=deg)
    _assert_close(got, want, f64, S, dg, what="mean, val=None")
    got2, _ = _run_gpu(rowptr, col, ones, x, np.zeros((M, F), np.float32), accumulate=False, row_div=deg, col_dtype=torch.int32)
    _assert_close(got2, want, f64, S, dg, what="mean, overwrite, int32 col")
    # with a non-zero previous value the division covers the whole sum, on every row
    init = rng.standard_normal((M, F), dtype=np.float32)
    w3 = init.copy(); orc.spmm_accumulate(rowptr, col, ones, x, w3); orc.row_divide(w3, deg)
    g3, _ = _run_gpu(rowptr, col, ones, x, init, accumulate=True, row_div=deg)
    _assert_close(g3, w3, orc.spmm_f64(rowptr, col, ones, x, init) / deg[:, None],
                  _abs_sum64(rowptr, col, ones, x, init) / deg[:, None], dg, what="mean on accumulate")


def test_duplicates_linearity_and_transpose():
    M, K, F = 500, 400, 128
    rowptr, col, _ = random_csr(M, K, 9, seed=17, dup=True)
    rng = np.random.default_rng(2)
    vali = rng.integers(1, 4, col.shape).astype(np.float32)
    x1 = rng.integers(-8, 8, (K, F)).astype(np.float32)
    x2 = rng.integers(-8, 8, (K, F)).astype(np.float32)
    z = np.zeros((M, F), np.float32)
    A = sp.csr_matrix((vali, col, rowptr), shape=(M, K))  # sums duplicate entries
    g1, _ = _run_gpu(rowptr, col, vali, x1, z, True)
    g2, _ = _run_gpu(rowptr, col, vali, x2, z, True)
    g12, _ = _run_gpu(rowptr, col, vali, x1 + x2, z, True)
    assert np.array_equal(g1, (A @ x1).astype(np.float32))  # integer data: exact
    assert np.array_equal(g12, g1 + g2)
    # SPMM_backward == SPMM_forward on the transpose
    from super_gnn_amd import SparseTensor, SPMM_forward, SPMM_backward
    st = SparseTensor(rowptr=torch.from_numpy(rowptr), col=torch.from_numpy(col), value=torch.from_numpy(vali),
                      sparse_sizes=(M, K), is_sorted=True).cuda()
    g = torch.from_numpy(rng.integers(-8, 8, (M, F)).astype(np.float32)).cuda()
    og = torch.zeros(K, F, device="cuda")
    assert SPMM_backward(st, g, og) is None
    assert np.array_equal(og.cpu().numpy(), (A.T @ g.cpu().numpy()).astype(np.float32))
    o = torch.zeros(M, F, device="cuda")
    assert SPMM_forward(st, torch.from_numpy(x1).cuda(), o) is None
    assert np.array_equal(o.cpu().numpy(), g1)


def test_reference_test_recipe_cpu_tensors():
    # tests/test_spmm.py:69-114 of the reference, CPU tensors in, result copied back
    from super_gnn_amd import SparseTensor, SPMM_forward, SPMM_backward
    A = sp.random(20020, 1020, density=0.0007, format="csr", dtype=np.float32, random_state=0)
    src = SparseTensor.from_scipy(A).requires_grad_()
    other = torch.rand(1020, 128)
    out = torch.zeros(20020, 128)
    SPMM_forward(src, other, out)
    assert torch.allclose(torch.from_numpy(A @ other.numpy()), out, atol=1e-5)
    grad_out = torch.randn(20020, 128)
    other_grad = torch.zeros(1020, 128)
    SPMM_backward(src, grad_out, other_grad)
    want = torch.from_numpy(A.T.tocsr() @ grad_out.numpy())
    assert torch.allclose(want, other_grad, atol=1e-4, rtol=1e-5)
    ref = np.zeros((1020, 128), np.float32)
    AT = A.T.tocsr(); AT.sort_indices()
    orc.spmm_accumulate(AT.indptr.astype(np.int64), AT.indices.astype(np.int64), AT.data, grad_out.numpy(), ref)
    _assert_close(other_grad.numpy(), ref, what="backward vs oracle")


def test_reference_dispatch_rule_through_supergnn_ops():
    ops = _gpu()
    M, K, F = 2000, 3000, 300   # sparsity <= 1e-4 and F > 256 -> the reference overwrites
    rowptr, col, val = random_csr(M, K, 0.25, seed=4)
    rng = np.random.default_rng(4)
    x = rng.standard_normal((K, F), dtype=np.float32)
    junk = rng.standard_normal((M, F), dtype=np.float32)
    want = junk.copy(); orc.spmm_dispatch(rowptr, col, val, x, want)
    out = torch.from_numpy(junk.copy()).cuda()
    ops.spmm(torch.from_numpy(rowptr).cuda(), torch.from_numpy(col).cuda(), torch.from_numpy(val).cuda(),
             torch.from_numpy(x).cuda(), out, M, torch.empty(0, dtype=torch.int32), torch.empty(0, dtype=torch.int32))
    _assert_close(out.cpu().numpy(), want, what="dispatch")
    assert np.all(out.cpu().numpy()[np.diff(rowptr) == 0] == 0)


def test_errors_are_loud():
    ops = _gpu()
    dev = "cuda:0"
    rowptr = torch.tensor([0, 2, 3], dtype=torch.int64, device=dev)
    with pytest.raises(IndexError):
        ops.SpmmPlan(rowptr, torch.tensor([0, 5, 1], dtype=torch.int64, device=dev), 3)  # col 5 >= K
    with pytest.raises(IndexError):
        ops.SpmmPlan(torch.tensor([0, 3, 2], dtype=torch.int64, device=dev), torch.tensor([0, 1], dtype=torch.int64, device=dev), 3)
    plan = ops.SpmmPlan(rowptr, torch.tensor([0, 2, 1], dtype=torch.int64, device=dev), 3)
    x = torch.zeros(3, 8, device=dev); out = torch.zeros(2, 8, device=dev)
    with pytest.raises(TypeError):
        plan.run(torch.ones(3, dtype=torch.float64, device=dev), x, out)
    with pytest.raises(ValueError):
        plan.run(torch.ones(3, device=dev), torch.zeros(4, 8, device=dev), out)
    with pytest.raises(TypeError):
        ops.spmm(rowptr, torch.tensor([0, 2, 1], device=dev), None, x, out, 2, None, None)
    # empty matrix and matrix of empty rows are fine
    p0 = ops.SpmmPlan(torch.zeros(4, dtype=torch.int64, device=dev), torch.empty(0, dtype=torch.int64, device=dev), 3)
    o = torch.ones(3, 8, device=dev)
    p0.run(None, x, o, accumulate=True); assert bool((o == 1).all())
    p0.run(None, x, o, accumulate=False); assert bool((o == 0).all())


def test_power_law_graph_weighted_and_mean():
    # a scaled-down headline case: R-MAT graph, GCN-normalised weights, F = 128
    from super_gnn_amd import synth
    n = 60000
    rowptr_t, col_t = synth.rmat_graph(n, 700000, seed=1)
    w_t = synth.gcn_norm_weights(rowptr_t, col_t)
    rowptr, col, w = rowptr_t.numpy(), col_t.numpy().astype(np.int64), w_t.numpy()
    x = torch.randn(n, 128, generator=torch.Generator().manual_seed(2)).numpy()
    z = np.zeros((n, 128), np.float32)
    want = z.copy(); orc.spmm_accumulate(rowptr, col, w, x, want)
    f64 = orc.spmm_f64(rowptr, col, w, x)
    dg = np.diff(rowptr)
    got, plan = _run_gpu(rowptr, col, w, x, z, accumulate=True, col_dtype=torch.int32)
    assert plan.info()["long_rows"] > 0
    _assert_close(got, want, f64, _abs_sum64(rowptr, col, w, x), dg, what="rmat weighted")
    short = dg <= plan.info()["long_row_threshold"]
    assert np.array_equal(got[short], want[short])
    deg = np.maximum(np.diff(rowptr), 1).astype(np.float32)
    ones = np.ones_like(w)
    want_m = z.copy(); orc.spmm_accumulate(rowptr, col, ones, x, want_m); orc.row_divide(want_m, deg)
    got_m, _ = _run_gpu(rowptr, col, None, x, z, accumulate=True, row_div=deg, col_dtype=torch.int32)
    _assert_close(got_m, want_m, orc.spmm_f64(rowptr, col, ones, x) / deg[:, None],
                  _abs_sum64(rowptr, col, ones, x) / deg[:, None], dg, what="rmat mean")


@pytest.mark.parametrize("mode", ["0", "1", None])
def test_long_row_modes_agree_and_auto_choice(mode, monkeypatch):
    """Long rows are either regrouped by column class or cut in CSR order; both must meet the same
    bar, and the automatic choice must regroup a power-law graph and leave a uniform one alone."""
    from super_gnn_amd import synth
    if mode is None:
        monkeypatch.delenv("SGNN_SPMM_PARTITION", raising=False)
    else:
        monkeypatch.setenv("SGNN_SPMM_PARTITION", mode)
    n = 40000
    rp_t, col_t = synth.rmat_graph(n, 500000, seed=3)
    rowptr, col = rp_t.numpy(), col_t.numpy().astype(np.int64)
    rng = np.random.default_rng(0)
    val = rng.random(col.shape[0], dtype=np.float32)
    x = rng.standard_normal((n, 64), dtype=np.float32)
    z = np.zeros((n, 64), np.float32)
    want = z.copy(); orc.spmm_accumulate(rowptr, col, val, x, want)
    got, plan = _run_gpu(rowptr, col, val, x, z, accumulate=True)
    info = plan.info()
    assert info["long_rows"] > 0
    assert info["partitioned"] == (0 if mode == "0" else 1)
    _assert_close(got, want, orc.spmm_f64(rowptr, col, val, x), _abs_sum64(rowptr, col, val, x), np.diff(rowptr), what=f"mode {mode}")
    if mode is None:
        # uniform popularity over many columns: left in CSR order
        M, K = 3000, 2000000
        rowptr_u = np.arange(M + 1, dtype=np.int64) * 600
        col_u = np.sort(rng.integers(0, K, (M, 600)), axis=1).reshape(-1).astype(np.int64)
        val_u = rng.random(col_u.shape[0], dtype=np.float32)
        xu = rng.standard_normal((K, 4), dtype=np.float32)
        zu = np.zeros((M, 4), np.float32)
        wu = zu.copy(); orc.spmm_accumulate(rowptr_u, col_u, val_u, xu, wu)
        gu, plan_u = _run_gpu(rowptr_u, col_u, val_u, xu, zu, accumulate=True)
        assert plan_u.info()["partitioned"] == 0 and 0 < plan_u.info()["top_share_ppm"] < 100000
        _assert_close(gu, wu, orc.spmm_f64(rowptr_u, col_u, val_u, xu), _abs_sum64(rowptr_u, col_u, val_u, xu), np.diff(rowptr_u), what="uniform")


def _cpu_runnable_case():
    """The small reference-runnable configuration: 10 000 nodes, 16 random neighbours + a self loop
    per row (sorted, duplicates kept), unit weights, 10 000 x 128 N(0,1) features, sum into zeros."""
    N = 10_000
    g = torch.Generator().manual_seed(0)
    col = torch.randint(0, N, (N, 16), generator=g)
    col = torch.sort(torch.cat([col, torch.arange(N).unsqueeze(1)], dim=1), dim=1).values.reshape(-1)
    rowptr = 17 * torch.arange(N + 1, dtype=torch.int64)
    x = torch.randn(N, 128, generator=g)
    return rowptr, col, torch.ones(col.numel()), x, g


def test_cpu_runnable_configuration_is_bit_identical():
    """Every row has 17 edges (short-row path): the GPU performs the reference's fma chain, so the
    result equals the CPU restatement bit for bit, through the reference's own call signature."""
    from super_gnn_amd import SparseTensor, SPMM_forward
    rowptr, col, val, x, _ = _cpu_runnable_case()
    want = np.zeros((10_000, 128), np.float32)
    orc.spmm_accumulate(rowptr.numpy(), col.numpy(), val.numpy(), x.numpy(), want)
    adj = SparseTensor(rowptr=rowptr, col=col, value=val, sparse_sizes=(10_000, 10_000)).cuda()
    out = torch.zeros(10_000, 128, device="cuda")
    SPMM_forward(adj, x.cuda(), out)
    assert np.array_equal(out.cpu().numpy(), want)
    ref = orc.ref_ops()
    if ref is not None:   # the reference's own x86 extension, when it was built on this host
        got = torch.zeros(10_000, 128)
        T = torch.get_num_threads()     # the reference reads one row range per OpenMP thread (spmm.cpp:408)
        split = torch.tensor([10_000 * t // T for t in range(T + 1)], dtype=torch.int32)
        ref.spmm(rowptr, col, val, x, got, 10_000, split, torch.tensor([0, 128], dtype=torch.int32))
        assert np.array_equal(got.numpy(), want)


def test_bound_values_follow_in_place_changes():
    """Values bound to the plan (second use of the same tensor) give the same bits as unbound ones,
    and an in-place change of the tensor is picked up by the very next call."""
    ops = _gpu()
    rowptr, col, val = random_csr(600, 500, 8, seed=77, empty_frac=0.1, hubs=6, hub_deg=900)
    x = np.random.default_rng(1).standard_normal((500, 64)).astype(np.float32)
    dev = torch.device("cuda:0")
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), 500, long_row_threshold=32)
    assert plan.info()["long_rows"] > 0
    v, xd = torch.from_numpy(val).to(dev), torch.from_numpy(x).to(dev)
    outs = []
    for _ in range(3):               # call 1 unbound, call 2 binds, call 3 uses the bound copy
        o = torch.zeros(600, 64, device=dev)
        plan.run(v, xd, o, accumulate=True)
        outs.append(o)
    assert plan._bound is not None and plan._bound[0] is v
    o = torch.zeros(600, 64, device=dev)
    plan.run(v[:], xd, o, accumulate=True)      # a view of the bound tensor: still bound, same bits
    assert plan._bound[0] is v and torch.equal(o, outs[0])
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    v.mul_(-2.0)                     # in place: same tensor, new version
    o = torch.zeros(600, 64, device=dev)
    plan.run(v, xd, o, accumulate=True)
    assert torch.equal(o, -2.0 * outs[0])
    v2 = v.clone()                   # another tensor: unbound path, same result
    o2 = torch.zeros(600, 64, device=dev)
    plan.run(v2, xd, o2, accumulate=True)
    assert torch.equal(o2, o)


@pytest.mark.parametrize("F,row_blocks", [(128, False), (602, False), (100, True)])
def test_steady_state_calls_replay_from_a_captured_graph(F, row_blocks, monkeypatch):
    """After warm-up a call only launches kernels (no allocation, no synchronisation), so an
    SpMM + quantize + fused-SpMM sequence can be captured once and replayed; every replay, with eager
    work in between, must reproduce the eager result bit for bit.  F = 602: rows on 8-byte boundaries (unaligned
    vector loads, packed bytes staged through LDS, two-code lanes in the fused product); row_blocks: the plan
    held as several row blocks."""
    ops = _gpu()
    dev = torch.device("cuda:0")
    rowptr, col, val = random_csr(4000, 3000, 9, seed=5, empty_frac=0.2, hubs=8, hub_deg=1200)
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(3000, F, generator=gen).to(dev)
    if row_blocks:
        monkeypatch.setenv("SGNN_SPMM_PART_EDGES", str(int(rowptr[-1]) // 3))
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), 3000)
    monkeypatch.delenv("SGNN_SPMM_PART_EDGES", raising=False)
    v = torch.from_numpy(val).to(dev)
    seg = torch.tensor([0, 1001, 2003, 3000], dtype=torch.int32)
    segs = ops.quant_segments(seg, 4)
    q = torch.zeros(segs.n_packed, F, dtype=torch.uint8, device=dev)
    prm = torch.zeros(3000, 2, device=dev)
    out, out_q = torch.zeros(4000, F, device=dev), torch.zeros(4000, F, device=dev)

    def step():
        out.zero_(); out_q.zero_()
        plan.run(v, x, out, accumulate=True)
        ops.quantize_tensor_for_all_procs(x, q, prm, seg, 3, 4)
        plan.run_quantized(v, q, prm, segs, 4, out_q, accumulate=True)

    for _ in range(3):          # warm-up: lazy work lists, partial buffer, value and slot binding
        step()
    torch.cuda.synchronize()
    want, want_q = out.clone(), out_q.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for i in range(4):
        out.fill_(float(i)); out_q.fill_(-1.0); q.zero_()          # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want) and torch.equal(out_q, want_q), f"replay {i}"


def test_workgroup_per_hub_row_alternative(monkeypatch):
    # the scheduling kept for comparison (one workgroup per long row, partial sums reduced in LDS): same bar
    ops = _gpu()
    dev = torch.device("cuda:0")
    monkeypatch.setenv("SGNN_SPMM_HUB_LDS", "1")
    for F in (128, 100, 602, 7):
        rowptr, col, val = random_csr(1200, 900, 10, seed=F, empty_frac=0.2, hubs=6, hub_deg=2000, dup=True)
        x = np.random.default_rng(F).standard_normal((900, F)).astype(np.float32)
        init = np.random.default_rng(F + 1).standard_normal((1200, F)).astype(np.float32)
        div = np.maximum(np.diff(rowptr), 1).astype(np.float32)
        plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), 900)
        for accumulate, mean in ((True, False), (False, True)):
            out = torch.from_numpy(init.copy()).to(dev)
            plan.run(torch.from_numpy(val).to(dev), torch.from_numpy(x).to(dev), out, accumulate=accumulate,
                     row_div=torch.from_numpy(div).to(dev) if mean else None)
            base = init if accumulate else None
            want = init.copy() if accumulate else np.zeros_like(init)
            orc.spmm_accumulate(rowptr, col, val, x, want)
            f64, asum = orc.spmm_f64(rowptr, col, val, x, base), _abs_sum64(rowptr, col, val, x, base)
            if mean:
                orc.row_divide(want, div)
                f64, asum = f64 / div[:, None].astype(np.float64), asum / div[:, None].astype(np.float64)
            _assert_close(out.cpu().numpy(), want, f64, asum, np.diff(rowptr), what=f"hub rows in LDS, F={F}")


def test_explicit_rebinding_after_an_edit_the_version_counter_does_not_see():
    ops = _gpu()
    dev = torch.device("cuda:0")
    rowptr, col, val = random_csr(600, 500, 8, seed=13, hubs=3, hub_deg=400)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), 500)
    x = torch.randn(500, 32, generator=torch.Generator().manual_seed(2)).to(dev)
    w = torch.from_numpy(val).to(dev)
    out = torch.zeros(600, 32, device=dev)
    for _ in range(3):                                   # bound from the second call on
        out.zero_(); plan.run(w, x, out, accumulate=True)
    first = out.clone()
    w.data.mul_(3.0)                                     # the version counter stays where it was
    plan.bind_values(w)
    out.zero_(); plan.run(w, x, out, accumulate=True)
    want = np.zeros((600, 32), np.float32)
    orc.spmm_accumulate(rowptr, col, w.cpu().numpy(), x.cpu().numpy(), want)
    _assert_close(out.cpu().numpy(), want, orc.spmm_f64(rowptr, col, w.cpu().numpy(), x.cpu().numpy(), None),
                      _abs_sum64(rowptr, col, w.cpu().numpy(), x.cpu().numpy(), None), np.diff(rowptr), what="rebound")
    assert not torch.equal(out, first)
    plan.unbind_values()
    out2 = torch.zeros(600, 32, device=dev); plan.run(w, x, out2, accumulate=True)
    assert torch.equal(out2, out)                        # same floats with and without the bound copy


def test_plan_finalised_during_a_capture_does_not_invalidate_it():
    """Python may run a dead plan's finaliser at any time, also inside someone's graph capture; freeing device
    memory there would invalidate the capture, so the wrapper parks the handle until later."""
    import gc
    ops = _gpu()
    dev = torch.device("cuda:0")
    rowptr, col, val = random_csr(500, 400, 7, seed=11, hubs=2, hub_deg=300)
    rp, cl = torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev)
    x = torch.randn(400, 64, generator=torch.Generator().manual_seed(1)).to(dev)
    v = torch.from_numpy(val).to(dev)
    out = torch.zeros(500, 64, device=dev)
    plan = ops.SpmmPlan(rp, cl, 400)
    for _ in range(3):
        out.zero_(); plan.run(v, x, out, accumulate=True)
    torch.cuda.synchronize()
    want = out.clone()

    class Holder:
        pass
    gc.collect()                                                      # leftovers of earlier tests go now
    h = Holder(); h.me = h; h.plan = ops.SpmmPlan(rp, cl, 400)      # a plan only the cyclic collector can reach
    h.plan.run(v, x, torch.zeros(500, 64, device=dev), accumulate=True)
    torch.cuda.synchronize()
    del h
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gc.collect()                                                  # the dead plan's finaliser runs here
        out.zero_(); plan.run(v, x, out, accumulate=True)
    assert len(ops._deferred_handles) == 1
    for i in range(2):
        out.fill_(3.0); torch.cuda.synchronize()
        graph.replay(); torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i}"
    ops.SpmmPlan(rp, cl, 400)                                         # creating a plan releases the parked handle
    assert not ops._deferred_handles


@pytest.mark.parametrize("tag", ["spmm_acc", "spmm_acc128", "spmm_ovw"])
def test_committed_reference_extension_vectors(tag):
    # inputs and the outputs the reference's own x86 extension produced for them (tests/golden/make_ref_vectors.py);
    # needs neither the reference checkout nor AVX-512 on the test host
    import os
    RV = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz"))
    ops = _gpu()
    rowptr, col, val, x, init, want = (RV[f"{tag}_{k}"] for k in ("rowptr", "col", "val", "x", "init", "out"))
    M, F = init.shape
    out = torch.from_numpy(init.copy())
    # CPU tensors in, the reference's own dispatch rule decides accumulate / overwrite
    ops.spmm(torch.from_numpy(rowptr), torch.from_numpy(col), torch.from_numpy(val), torch.from_numpy(x), out, M)
    got = out.numpy()
    if tag == "spmm_ovw":
        assert ops.reference_overwrites(col.shape[0], M, x.shape[0], F)
        np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-7)  # mul+add vs fma is build dependent in that branch
        assert np.all(got[np.diff(rowptr) == 0] == 0)
    else:
        assert np.array_equal(got, want), "short rows: the reference's fma sequence, bit for bit"


def test_full_size_graph_exact_on_small_integers():
    # The headline shape (2.45 M nodes, ~62 M edges, F = 128).  With small integer features and weights every
    # partial sum is an integer below 2^24, so fp32 addition is exact in any order and the product has ONE
    # right answer: the kernels (short rows, class-regrouped long rows, final sums, mean epilogue, transpose)
    # must reproduce it bit for bit.  The expected values are accumulated in fp64 with index_add_.
    from super_gnn_amd import synth
    ops = _gpu()
    dev = torch.device("cuda:0")
    n, F = 2_450_000, 128
    rowptr, col = synth.rmat_graph(n, 31_000_000, seed=1, device=dev)
    nnz = int(col.numel())
    g = torch.Generator(device=dev); g.manual_seed(11)
    w = torch.randint(1, 3, (nnz,), generator=g, device=dev).float()
    x = torch.randint(-4, 5, (n, F), generator=g, device=dev).float()
    deg = rowptr[1:] - rowptr[:-1]
    assert int(deg.max()) * 8 < 2 ** 24
    rows = torch.repeat_interleave(torch.arange(n, device=dev), deg)

    def expected(init):
        want = init.double()
        step = 1 << 22
        for e0 in range(0, nnz, step):
            e1 = min(nnz, e0 + step)
            want.index_add_(0, rows[e0:e1], x[col[e0:e1]].double() * w[e0:e1, None].double())
        return want

    plan = ops.SpmmPlan(rowptr, col.to(torch.int32), n)
    info = plan.info()
    assert info["long_rows"] > 1000 and info["partitioned"] == 1
    init = torch.randint(-3, 4, (n, F), generator=g, device=dev).float()
    want = expected(init)
    out = init.clone()
    plan.run(w, x, out, accumulate=True)
    assert torch.equal(out.double(), want)
    # a second call takes the bound-weights path for the long rows: same answer
    out2 = init.clone()
    plan.run(w, x, out2, accumulate=True)
    assert torch.equal(out2, out)
    # overwrite mode + mean epilogue: (A x) / max(deg, 1), one correctly rounded division per element
    div = deg.clamp(min=1).float()
    out3 = torch.full((n, F), 7.0, device=dev)
    plan.run(w, x, out3, accumulate=False, row_div=div)
    want3 = (want - init.double()).float() / div[:, None]
    assert torch.equal(out3, want3)
    del want, want3, out2, out3
    # the fused int8 path on the same graph: rows quantized with scale 1 decode to the integers again
    seg = torch.tensor([0, n], dtype=torch.int32)
    q = torch.empty(n, F, dtype=torch.uint8, device=dev)
    p = torch.empty(n, 2, device=dev)
    x8 = x.clone(); x8[:, 0] = -100.0; x8[:, 1] = 155.0   # every row spans exactly 255 steps of 1.0
    ops.quantize_tensor_for_all_procs(x8, q, p, seg, 1, 8)
    assert bool((p[:, 1] == 1.0).all()) and bool((p[:, 0] == -100.0).all())
    d8 = torch.empty_like(x8)
    ops.dequantize_tensor_for_all_procs(q, d8, p, seg, 1, 8)
    assert torch.equal(d8, x8)
    w1 = torch.ones_like(w)   # keep the sums of the two wide columns below 2^24
    assert int(deg.max()) * 155 < 2 ** 24
    ref = torch.zeros(n, F, device=dev)
    plan.run(w1, x8, ref, accumulate=True)
    fused = torch.zeros(n, F, device=dev)
    plan.run_quantized(w1, q, p, ops.quant_segments(seg, 8), 8, fused, accumulate=True)
    assert torch.equal(fused, ref)


def test_full_size_community_graph_exact_on_small_integers():
    # The wide-feature configuration (233 k nodes, ~114 M edges, average degree ~490, F = 602: float2 lanes,
    # every row on the long-row path), mean aggregation, forward and transpose.  Exact for the same reason
    # as the test above.
    from super_gnn_amd import synth
    ops = _gpu()
    dev = torch.device("cuda:0")
    n, F = 233_000, 602
    rowptr, col = synth.sbm_graph(n, 50, 0.03048, 0.001524, seed=3, device=dev)
    nnz = int(col.numel())
    g = torch.Generator(device=dev); g.manual_seed(12)
    x = torch.randint(-4, 5, (n, F), generator=g, device=dev).float()
    deg = rowptr[1:] - rowptr[:-1]
    assert int(deg.max()) * 4 < 2 ** 24
    rows = torch.repeat_interleave(torch.arange(n, device=dev), deg)
    want = torch.zeros(n, F, dtype=torch.float64, device=dev)
    step = 1 << 20
    for e0 in range(0, nnz, step):
        e1 = min(nnz, e0 + step)
        want.index_add_(0, rows[e0:e1], x[col[e0:e1]].double())
    div = deg.clamp(min=1).float()
    plan = ops.SpmmPlan(rowptr, col.to(torch.int32), n)
    assert plan.info()["long_rows"] > n // 2
    out = torch.full((n, F), -1.0, device=dev)
    plan.run(None, x, out, accumulate=False, row_div=div)
    assert torch.equal(out, want.float() / div[:, None])
    # the graph is symmetric: the transpose product (backward) is the same matrix
    out_t = torch.zeros(n, F, device=dev)
    ops.SpmmPlan(rowptr, col, n).run(torch.ones(nnz, device=dev), x, out_t, accumulate=True)
    assert torch.equal(out_t.double(), want)


@pytest.mark.parametrize("F,pad_x,pad_o,off_x,off_o", [(128, 64, 32, 16, 8), (128, 3, 5, 1, 2), (602, 2, 6, 2, 4), (64, 0, 64, 0, 64)])
def test_leading_dimensions_through_the_c_abi(F, pad_x, pad_o, off_x, off_o):
    # X and out as column windows of wider matrices (ldx, ldo > F; aligned and unaligned starts): same bits as
    # the contiguous call, and nothing outside the window is written
    ops = _gpu()
    from super_gnn_amd._lib import lib, check
    dev = torch.device("cuda:0")
    M, K = 3000, 2500
    rowptr, col, val = random_csr(M, K, 9, seed=21, empty_frac=0.1, hubs=3, hub_deg=900)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    g = torch.Generator().manual_seed(22)
    xw = torch.randn(K, F + pad_x, generator=g).to(dev)
    ow = torch.randn(M, F + pad_o, generator=g).to(dev)
    w = torch.from_numpy(val).to(dev)
    div = torch.from_numpy(np.maximum(np.diff(rowptr), 1).astype(np.float32)).to(dev)
    for accumulate, row_div in ((1, None), (0, None), (1, div)):
        want = ow[:, off_o:off_o + F].contiguous()
        plan.run(w, xw[:, off_x:off_x + F].contiguous(), want, accumulate=bool(accumulate), row_div=row_div)
        got = ow.clone()
        check(lib.sgnn_spmm_csr_f32(plan._h, w.data_ptr(), xw.data_ptr() + 4 * off_x, got.data_ptr() + 4 * off_o, F,
                                    F + pad_x, F + pad_o, accumulate, row_div.data_ptr() if row_div is not None else None,
                                    torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert torch.equal(got[:, off_o:off_o + F], want)
        keep = torch.ones(F + pad_o, dtype=torch.bool, device=dev); keep[off_o:off_o + F] = False
        assert torch.equal(got[:, keep], ow[:, keep])


@pytest.mark.parametrize("F", [256, 320, 384, 1024, 2052])
def test_feature_slices_of_wide_products_change_nothing(F, monkeypatch):
    # wide fp32 products of large operands run one feature slice after the other (cache footprint of a gathered row);
    # forced here on a small matrix: same bits as the unsliced product in every mode, with long and empty rows, and
    # inside a padded window
    ops = _gpu()
    from super_gnn_amd._lib import lib, check
    dev = torch.device("cuda:0")
    M, K = 2000, 1800
    rowptr, col, val = random_csr(M, K, 7, seed=F, empty_frac=0.15, hubs=4, hub_deg=700)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    g = torch.Generator().manual_seed(F + 1)
    xw = torch.randn(K, F + 8, generator=g).to(dev)
    ow = torch.randn(M, F + 4, generator=g).to(dev)
    w = torch.from_numpy(val).to(dev)
    div = torch.from_numpy(np.maximum(np.diff(rowptr), 1).astype(np.float32)).to(dev)
    st = torch.cuda.current_stream().cuda_stream
    for accumulate, row_div, wv in ((1, None, w), (0, None, w), (1, div, None), (0, div, w)):
        outs = []
        for sl in ("0", "128", "172"):
            monkeypatch.setenv("SGNN_SPMM_SLICE", sl)
            got = ow.clone()
            check(lib.sgnn_spmm_csr_f32(plan._h, wv.data_ptr() if wv is not None else None, xw.data_ptr() + 16,
                                        got.data_ptr(), F, F + 8, F + 4, accumulate,
                                        row_div.data_ptr() if row_div is not None else None, st))
            torch.cuda.synchronize()
            outs.append(got)
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
        assert torch.equal(outs[1][:, F:], ow[:, F:])
    monkeypatch.setenv("SGNN_SPMM_SLICE", "64")
    x = xw[:, 4:4 + F].contiguous()
    init = np.zeros((M, F), dtype=np.float32)
    out = torch.zeros(M, F, device=dev)
    plan.run(w, x, out, accumulate=True)
    ref = init.copy(); orc.spmm_accumulate(rowptr, col, val, x.cpu().numpy(), ref)
    short = np.diff(rowptr) <= plan.info()["long_row_threshold"]
    assert np.array_equal(out.cpu().numpy()[short], ref[short])


def test_feature_slices_at_the_size_where_the_library_chooses_them(monkeypatch):
    # 1.0 M dense rows of 256 floats (1.02 GB): above the operand size from which the library slices by itself
    ops = _gpu()
    from super_gnn_amd import synth
    dev = torch.device("cuda:0")
    n, F = 1_000_000, 256
    rowptr, col = synth.rmat_graph(n, 6_000_000, a=0.57, b=0.19, c=0.19, seed=4, device=dev)
    w = synth.gcn_norm_weights(rowptr, col)
    plan = ops.SpmmPlan(rowptr, col, n)
    assert plan.info()["long_rows"] > 0
    g = torch.Generator(device=dev).manual_seed(9)
    x = torch.randn(n, F, generator=g, device=dev)
    init = torch.randn(n, F, generator=g, device=dev)
    outs = []
    for sl in (None, "0"):
        if sl is None:
            monkeypatch.delenv("SGNN_SPMM_SLICE", raising=False)
        else:
            monkeypatch.setenv("SGNN_SPMM_SLICE", sl)
        out = init.clone()
        plan.run(w, x, out, accumulate=True)
        torch.cuda.synchronize()
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
