"""Matrices held as row blocks (2^31 edges or more): the plan cuts the rows into consecutive blocks of fewer
edges, each a plan of its own, and every call runs the blocks in turn.  Checked two ways: with the block size
lowered through SGNN_SPMM_PART_EDGES the blocked plan must give the same bits as the single plan on every entry
point; and a matrix of more than 2^31 edges at its real size must equal the exact integer result."""
import ctypes

import numpy as np
import pytest
import torch

from _util import random_csr

pytestmark = pytest.mark.gpu


def _plans(monkeypatch, rowptr, col, K, cap, **kw):
    from super_gnn_amd import supergnn_ops as ops
    rp, cl = torch.from_numpy(rowptr).cuda(), torch.from_numpy(col).cuda()
    monkeypatch.delenv("SGNN_SPMM_PART_EDGES", raising=False)
    whole = ops.SpmmPlan(rp, cl, K, **kw)
    monkeypatch.setenv("SGNN_SPMM_PART_EDGES", str(cap))
    blocked = ops.SpmmPlan(rp, cl, K, **kw)
    monkeypatch.delenv("SGNN_SPMM_PART_EDGES", raising=False)
    return ops, whole, blocked


@pytest.mark.parametrize("case", range(8))
def test_row_blocks_equal_the_single_plan(case, monkeypatch):
    rng = np.random.default_rng(7000 + case)
    M, K = int(rng.integers(50, 3000)), int(rng.integers(20, 2500))
    F = int(rng.choice([8, 64, 100, 128, 602]))
    hubs = int(rng.integers(0, 4))
    rowptr, col, val = random_csr(M, K, float(rng.choice([1, 6, 30])), seed=7100 + case, empty_frac=float(rng.choice([0, 0.4])),
                                  hubs=hubs, hub_deg=int(rng.integers(200, 1500)))
    nnz = int(rowptr[-1])
    cap = max(int(np.diff(rowptr).max()), nnz // int(rng.integers(2, 9))) + 1
    ops, whole, blocked = _plans(monkeypatch, rowptr, col, K, cap, long_row_threshold=int(rng.choice([0, 32])))
    assert blocked.info()["nnz"] == nnz and blocked.info()["long_rows"] == whole.info()["long_rows"]
    g = torch.Generator().manual_seed(case)
    x = torch.randn(K, F, generator=g).cuda()
    init = torch.randn(M, F, generator=g).cuda()
    v = torch.from_numpy(val).cuda()
    div = torch.from_numpy(np.maximum(np.diff(rowptr), 1).astype(np.float32)).cuda()
    for w, accumulate, rd in ((v, True, None), (None, False, div), (v, True, div), (v, True, None)):  # the last repeat runs with bound values
        a, b = init.clone(), init.clone()
        whole.run(w, x, a, accumulate=accumulate, row_div=rd)
        blocked.run(w, x, b, accumulate=accumulate, row_div=rd)
        assert torch.equal(a, b)
    # the entry point that allocates nothing
    from super_gnn_amd import _lib
    a, b = init.clone(), init.clone()
    for plan, out in ((whole, a), (blocked, b)):
        _lib.check(_lib.lib.sgnn_spmm_csr_f32_noalloc(plan._h, v.data_ptr(), x.data_ptr(), out.data_ptr(), F, F, F, 1, None, ops._stream()))
    assert torch.equal(a, b)
    # fused unpack+dequantize+SpMM with ragged segments (per-edge slot streams live in the blocks)
    if F % 2 == 0:
        bits = int(rng.choice([8, 4, 2]))
        cuts = np.sort(rng.integers(0, K + 1, size=2))
        wr = torch.tensor([0, int(cuts[0]), int(cuts[1]), K], dtype=torch.int32)
        epb = 8 // bits
        npk = sum(-(-int(hi - lo) // epb) for lo, hi in zip(wr[:-1], wr[1:]))
        q = torch.zeros(npk, F, dtype=torch.uint8, device="cuda"); prm = torch.zeros(K, 2, device="cuda")
        ops.quantize_tensor_for_all_procs(x, q, prm, wr, 3, bits)
        segs = ops.quant_segments(wr, bits)
        a, b = init.clone(), init.clone()
        whole.run_quantized(v, q, prm, segs, bits, a, accumulate=True)
        blocked.run_quantized(v, q, prm, segs, bits, b, accumulate=True)
        assert torch.equal(a, b)


def test_row_blocks_share_one_restaged_operand(monkeypatch):
    """With the band schedule every block of a plan gathers from the same restaged copy of the dense operand: it is
    made once per product and held once, however many blocks there are (64 blocks of a 60 MB operand would
    otherwise hold 3.8 GB)."""
    M, K, F = 6000, 30000, 512
    rowptr, col, val = random_csr(M, K, 40, seed=77)
    monkeypatch.setenv("SGNN_SPMM_BAND", "1")
    ops, whole, blocked = _plans(monkeypatch, rowptr, col, K, int(rowptr[-1]) // 64 + 1)
    assert whole.schedule(F)["band"] == 1
    x = torch.randn(K, F, generator=torch.Generator().manual_seed(3)).cuda()
    init = torch.randn(M, F, generator=torch.Generator().manual_seed(4)).cuda()
    v = torch.from_numpy(val).cuda()
    a = init.clone()
    whole.run(v, x, a)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    b = init.clone()
    blocked.run(v, x, b)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert torch.equal(a, b)
    assert free0 - free1 < 4 * K * F * 4, f"the blocked plan took {(free0 - free1) >> 20} MB for its first product"
    x2 = x * 2.0                              # a new operand must be restaged, not taken from the last product
    a2, b2 = init.clone(), init.clone()
    whole.run(v, x2, a2); blocked.run(v, x2, b2)
    assert torch.equal(a2, b2) and not torch.equal(a2, a)


def test_plans_release_their_memory(monkeypatch):
    """Everything a plan allocates -- work lists, regrouped long rows, bound values and slot streams, the band
    schedule and its restaged operand, the row blocks -- goes back when the plan is destroyed."""
    import gc
    from super_gnn_amd import supergnn_ops as ops
    M, K, F = 5000, 20000, 256
    rowptr, col, val = random_csr(M, K, 30, seed=5, hubs=6, hub_deg=3000)
    rp, cl, v = torch.from_numpy(rowptr).cuda(), torch.from_numpy(col).cuda(), torch.from_numpy(val).cuda()
    x = torch.randn(K, F, generator=torch.Generator().manual_seed(1)).cuda()
    out = torch.zeros(M, F, device="cuda")
    seg = torch.tensor([0, 7001, K], dtype=torch.int32)
    segs = ops.quant_segments(seg, 2)
    q = torch.zeros(segs.n_packed, F, dtype=torch.uint8, device="cuda"); prm = torch.zeros(K, 2, device="cuda")
    ops.quantize_tensor_for_all_procs(x, q, prm, seg, 2, 2)

    def cycle(blocks, band):
        monkeypatch.setenv("SGNN_SPMM_BAND", "1" if band else "0")
        if blocks:
            monkeypatch.setenv("SGNN_SPMM_PART_EDGES", str(int(rowptr[-1]) // 5))
        plan = ops.SpmmPlan(rp, cl, K)
        monkeypatch.delenv("SGNN_SPMM_PART_EDGES", raising=False)
        for _ in range(2):
            plan.run(v, x, out)
            plan.run_quantized(v, q, prm, segs, 2, out)
        torch.cuda.synchronize()
        del plan
        gc.collect()

    cycle(True, True)                       # first use of every kernel: code objects, event pools
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for i in range(12):
        cycle(i % 2 == 0, i % 3 != 0)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free0 - free1 < 8 << 20, f"{(free0 - free1) >> 20} MB not returned after 12 plans"


def test_a_row_longer_than_a_block_is_refused(monkeypatch):
    from super_gnn_amd import supergnn_ops as ops
    rowptr, col, _ = random_csr(100, 400, 3, seed=1, hubs=1, hub_deg=300)
    monkeypatch.setenv("SGNN_SPMM_PART_EDGES", "200")
    with pytest.raises(Exception, match="more than one plan holds"):
        ops.SpmmPlan(torch.from_numpy(rowptr).cuda(), torch.from_numpy(col).cuda(), 400)


def test_more_than_two_to_the_31_edges_exact_on_small_integers():
    """1.05 M rows of 2048 edges and 2 M rows of 8 edges: 2,166,400,000 edges, 32-bit column indices (8.7 GB).
    Unit weights and features in {0..3}: every partial sum is a small integer, so any summation order gives the
    same fp32 result, which is compared with torch gathers row block by row block."""
    from super_gnn_amd import supergnn_ops as ops
    free, _ = torch.cuda.mem_get_info()
    if free < 80 * 2 ** 30:
        pytest.skip("needs about 60 GB of free device memory")
    ML, DL, MS, DS, K, F = 1_050_000, 2048, 2_000_000, 8, 300_000, 8
    g = torch.Generator(device="cuda"); g.manual_seed(11)
    col = torch.empty(ML * DL + MS * DS, dtype=torch.int32, device="cuda")
    step = 50_000
    for r in range(0, ML, step):   # filled in pieces: randint makes int64 first
        n = min(step, ML - r) * DL
        col[r * DL: r * DL + n] = torch.randint(0, K, (n,), generator=g, device="cuda").to(torch.int32)
    col[ML * DL:] = torch.randint(0, K, (MS * DS,), generator=g, device="cuda").to(torch.int32)
    rowptr = torch.cat([torch.arange(0, ML + 1, dtype=torch.int64, device="cuda") * DL,
                        ML * DL + torch.arange(1, MS + 1, dtype=torch.int64, device="cuda") * DS])
    nnz = int(rowptr[-1])
    assert nnz == col.numel() and nnz > 2 ** 31
    x = torch.randint(0, 4, (K, F), generator=g, device="cuda").float()
    plan = ops.SpmmPlan(rowptr, col, K)
    info = plan.info()
    assert info["nnz"] == nnz and info["long_rows"] == ML
    out = torch.ones(ML + MS, F, device="cuda")
    plan.run(None, x, out, accumulate=True)
    torch.cuda.synchronize()
    for r in range(0, ML, step):
        n = min(step, ML - r)
        want = 1.0 + x[col[r * DL:(r + n) * DL].long()].view(n, DL, F).sum(dim=1)
        assert torch.equal(out[r:r + n], want), f"long rows {r}..{r + n}"
    want = 1.0 + x[col[ML * DL:].long()].view(MS, DS, F).sum(dim=1)
    assert torch.equal(out[ML:], want)
