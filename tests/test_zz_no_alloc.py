"""sgnn_spmm_csr_f32_noalloc, the entry point for callers that cannot allocate device memory: it
must give the bits of sgnn_spmm_csr_f32 (which is itself checked against the oracle elsewhere in
this suite) while taking its long-row partial sums from the library's built-in scratch array.

Collected last on purpose (file name): the scratch array is shared state of the whole process, so
this also runs after every other test has used the library."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from _util import random_csr, assert_spmm_close, abs_sum64

pytestmark = pytest.mark.gpu


def _both(ops, lib, check, rowptr, col, val, x, init, accumulate, row_div):
    dev = torch.device("cuda:0")
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), x.shape[0])
    w = torch.from_numpy(val).to(dev)
    xd = torch.from_numpy(x).to(dev)
    div = torch.from_numpy(row_div).to(dev) if row_div is not None else None
    F = x.shape[1]
    st = torch.cuda.current_stream().cuda_stream
    outs = []
    for fn in (lib.sgnn_spmm_csr_f32, lib.sgnn_spmm_csr_f32_noalloc):
        out = torch.from_numpy(init.copy()).to(dev)
        check(fn(plan._h, w.data_ptr(), xd.data_ptr(), out.data_ptr(), F, F, F, int(accumulate),
                 div.data_ptr() if div is not None else None, st))
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
    return outs[0], outs[1], plan


def test_two_calls_in_a_row_second_one_smaller():
    import super_gnn_amd  # noqa: F401
    from super_gnn_amd import supergnn_ops as ops
    from super_gnn_amd._lib import lib, check
    # first call: hub rows whose partials fill a good part of the scratch; second call: a smaller
    # matrix and a narrower feature row, so stale partials of the first call lie right behind its own
    cases = [
        dict(M=6000, K=5000, F=256, deg=12, hubs=40, hub_deg=4000, seed=301, accumulate=True, mean=False),
        dict(M=900, K=700, F=100, deg=7, hubs=5, hub_deg=600, seed=302, accumulate=False, mean=True),
    ]
    for c in cases:
        rowptr, col, val = random_csr(c["M"], c["K"], c["deg"], seed=c["seed"], empty_frac=0.1, hubs=c["hubs"],
                                      hub_deg=c["hub_deg"])
        rng = np.random.default_rng(c["seed"])
        x = rng.standard_normal((c["K"], c["F"]), dtype=np.float32)
        init = rng.standard_normal((c["M"], c["F"]), dtype=np.float32)
        deg = np.diff(rowptr)
        row_div = np.maximum(deg, 1).astype(np.float32) if c["mean"] else None
        print(f"case {c}", flush=True)
        want, got, plan = _both(ops, lib, check, rowptr, col, val, x, init, c["accumulate"], row_div)
        assert plan.info()["long_rows"] == c["hubs"] and plan.info()["pieces"] > 0
        assert np.array_equal(got, want), "the non-allocating entry point must give the allocating one's bits"
        # and both against the CPU oracle, to the fp32 SpMM bar
        ref = init.copy() if c["accumulate"] else np.zeros_like(init)
        orc.spmm_accumulate(rowptr, col, val, x, ref)
        f64 = orc.spmm_f64(rowptr, col, val, x, init if c["accumulate"] else None)
        asum = abs_sum64(rowptr, col, val, x, init if c["accumulate"] else None)
        if row_div is not None:
            ref = ref / row_div[:, None]
            f64 = f64 / row_div[:, None].astype(np.float64)
            asum = asum / row_div[:, None].astype(np.float64)
        assert_spmm_close(got, ref, f64=f64, abs_sum=asum, deg=deg, what=f"noalloc F={c['F']}")


def test_refuses_what_does_not_fit_the_scratch():
    import super_gnn_amd  # noqa: F401
    from super_gnn_amd import supergnn_ops as ops
    from super_gnn_amd._lib import lib
    dev = torch.device("cuda:0")
    rowptr, col, val = random_csr(3000, 40000, 3, seed=303, hubs=400, hub_deg=30000)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), 40000)
    F = 256
    assert plan.info()["pieces"] * F * 4 > 64 << 20
    x = torch.zeros(40000, F, device=dev)
    out = torch.full((3000, F), 3.0, device=dev)
    w = torch.from_numpy(val).to(dev)
    rc = lib.sgnn_spmm_csr_f32_noalloc(plan._h, w.data_ptr(), x.data_ptr(), out.data_ptr(), F, F, F, 1, None,
                                       torch.cuda.current_stream().cuda_stream)
    assert rc == -1 and b"scratch" in lib.sgnn_last_error()
    torch.cuda.synchronize()
    assert bool((out == 3.0).all()), "a refused call must not have launched anything"
    # a narrower product of the same plan fits again
    F2 = 8
    if plan.info()["pieces"] * F2 * 4 <= 64 << 20:
        x2 = torch.ones(40000, F2, device=dev)
        o1 = torch.zeros(3000, F2, device=dev)
        o2 = torch.zeros(3000, F2, device=dev)
        st = torch.cuda.current_stream().cuda_stream
        assert lib.sgnn_spmm_csr_f32(plan._h, w.data_ptr(), x2.data_ptr(), o1.data_ptr(), F2, F2, F2, 1, None, st) == 0
        assert lib.sgnn_spmm_csr_f32_noalloc(plan._h, w.data_ptr(), x2.data_ptr(), o2.data_ptr(), F2, F2, F2, 1, None, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(o1, o2)


def _call(lib, check, fn, plan, w, x, out, F, accumulate=1, div=None):
    check(fn(plan._h, w.data_ptr() if w is not None else None, x.data_ptr(), out.data_ptr(), F, F, F, accumulate,
             div.data_ptr() if div is not None else None, torch.cuda.current_stream().cuda_stream))


def test_allocates_nothing_and_replays_from_a_captured_graph():
    import super_gnn_amd  # noqa: F401
    from super_gnn_amd import supergnn_ops as ops
    from super_gnn_amd._lib import lib, check
    dev = torch.device("cuda:0")
    M, K, F = 5000, 4000, 128
    rowptr, col, val = random_csr(M, K, 15, seed=311, empty_frac=0.1, hubs=30, hub_deg=3000)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    w = torch.from_numpy(val).to(dev)
    x = torch.randn(K, F, generator=torch.Generator().manual_seed(1)).to(dev)
    want = torch.zeros(M, F, device=dev)
    _call(lib, check, lib.sgnn_spmm_csr_f32, plan, w, x, want, F)
    out = torch.zeros(M, F, device=dev)
    _call(lib, check, lib.sgnn_spmm_csr_f32_noalloc, plan, w, x, out, F)      # warm
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        out.zero_()
        _call(lib, check, lib.sgnn_spmm_csr_f32_noalloc, plan, w, x, out, F)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "device memory moved during non-allocating calls"
    assert torch.equal(out, want)
    # under capture (an allocation or a lazy symbol lookup would invalidate the capture), then replays with eager work between
    graph = torch.cuda.CUDAGraph()
    gout = torch.zeros(M, F, device=dev)
    with torch.cuda.graph(graph):
        gout.zero_()
        _call(lib, check, lib.sgnn_spmm_csr_f32_noalloc, plan, w, x, gout, F)
    for i in range(3):
        gout.fill_(float(i + 7))
        out.normal_()                 # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(gout, want), f"replay {i}"


@pytest.mark.parametrize("switch,value,F", [("SGNN_SPMM_BAND", "1", 602), ("SGNN_SPMM_BAND", "1", 128),
                                              ("SGNN_SPMM_SLICE", "128", 256), ("SGNN_SPMM_PART_EDGES", "20000", 64)])
def test_other_schedules_through_the_non_allocating_entry_point(switch, value, F, monkeypatch):
    """Band schedule (taken here only once the allocating entry point has built it), feature slices (the scratch limit
    applies per slice) and row-block plans: the non-allocating call gives the allocating call's bits."""
    import super_gnn_amd  # noqa: F401
    from super_gnn_amd import supergnn_ops as ops
    from super_gnn_amd._lib import lib, check
    dev = torch.device("cuda:0")
    monkeypatch.setenv(switch, value)
    if switch == "SGNN_SPMM_BAND":
        monkeypatch.setenv("SGNN_SPMM_BAND_COLS", "200")
    M, K = 3000, 2500
    rowptr, col, val = random_csr(M, K, 20, seed=F, empty_frac=0.1, hubs=12, hub_deg=2000)
    deg = np.diff(rowptr)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
    w = torch.from_numpy(val).to(dev)
    xn = np.random.default_rng(F).standard_normal((K, F), dtype=np.float32)
    x = torch.from_numpy(xn).to(dev)
    short = torch.from_numpy(deg <= 128).to(dev)
    if switch == "SGNN_SPMM_BAND":
        # nothing built yet: the row-class kernels answer -- reference order on short rows, the fp32 bar on long ones
        first = torch.zeros(M, F, device=dev)
        _call(lib, check, lib.sgnn_spmm_csr_f32_noalloc, plan, w, x, first, F)
        ref = np.zeros((M, F), np.float32)
        orc.spmm_accumulate(rowptr, col, val, xn, ref)
        assert np.array_equal(first.cpu().numpy()[deg <= 128], ref[deg <= 128])
        assert_spmm_close(first.cpu().numpy(), ref, orc.spmm_f64(rowptr, col, val, xn, None), abs_sum64(rowptr, col, val, xn, None),
                          deg, what="noalloc before the band schedule exists")
    want = torch.zeros(M, F, device=dev)
    _call(lib, check, lib.sgnn_spmm_csr_f32, plan, w, x, want, F)          # builds what the schedule needs
    got = torch.zeros(M, F, device=dev)
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    _call(lib, check, lib.sgnn_spmm_csr_f32_noalloc, plan, w, x, got, F)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "device memory moved during the non-allocating call"
    assert torch.equal(got, want), f"{switch}={value}, F={F}"
    assert torch.equal(got[short], want[short])
    if switch == "SGNN_SPMM_BAND":
        assert plan.schedule(F)["band"] == 1
        ref = np.zeros((M, F), np.float32)
        orc.spmm_accumulate(rowptr, col, val, xn, ref)
        assert np.array_equal(got.cpu().numpy(), ref), "band schedule through the non-allocating call: CSR order on every row"
