"""GPU parity of the fused unpack+dequantize+SpMM path (remote boundary rows arrive packed).

Checked three ways: (1) bit-identical to the separate GPU path "unpack+dequantize, then SpMM" with
the same plan; (2) against the CPU oracle chain quant_rows -> dequant_rows -> spmm_accumulate within
the SpMM tolerance; (3) the pre/post-aggregation data flow of super_gnn/aggregator.py:61-93 at a
scaled-down size (local SpMM, then remote rows accumulated onto the same out)."""
import numpy as np
import pytest
import torch

from oracle import oracle as orc
from _util import random_csr, abs_sum64, assert_spmm_close

pytestmark = pytest.mark.gpu


def _setup(M, K, F, deg, bits, seg, seed, hubs=0):
    import super_gnn_amd  # noqa: F401
    from super_gnn_amd import supergnn_ops as ops
    rowptr, col, val = random_csr(M, K, deg, seed=seed, empty_frac=0.1, hubs=hubs, hub_deg=min(K * 2, 1500))
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(K, F, generator=g)
    x[::7] *= 30.0
    seg_t = torch.tensor(seg, dtype=torch.int32)
    P = seg_t.numel() - 1
    npk = int(orc.packed_rows(seg, bits).sum())
    q = torch.zeros(npk, F, dtype=torch.uint8, device="cuda")
    params = torch.zeros(K, 2, device="cuda")
    ops.quantize_tensor_for_all_procs(x.cuda(), q, params, seg_t, P, bits)
    plan = ops.SpmmPlan(torch.from_numpy(rowptr).cuda(), torch.from_numpy(col).cuda(), K)
    return ops, plan, rowptr, col, val, x, seg_t, P, q, params


@pytest.mark.parametrize("bits", [8, 4, 2])
@pytest.mark.parametrize("M,K,F,deg,seg,hubs", [
    (800, 600, 128, 9, [0, 600], 0),
    (800, 600, 128, 9, [0, 600], 4),                  # long rows: class-partitioned pieces
    (500, 403, 128, 7, [0, 5, 5, 130, 131, 403], 2),   # ragged segments: the row -> slot table is needed
    (300, 256, 256, 6, [0, 100, 256], 0),             # full wavefront per row; segment sizes divisible by 4
    (300, 250, 64, 6, [0, 33, 250], 1),               # 16-lane groups
    (200, 180, 1024, 4, [0, 180], 0),                 # 4 words per lane
    (150, 120, 100, 5, [0, 61, 120], 0),              # partly idle group
    (120, 90, 8, 5, [0, 90], 0),
    (400, 350, 602, 8, [0, 350], 3),                  # even width that is not a multiple of four: two-code lanes, five per lane
    (300, 256, 130, 6, [0, 100, 256], 2),             # two-code lanes, two per lane, ragged segments
    (200, 180, 6, 5, [0, 61, 180], 1),                # three two-code lanes
    (100, 90, 1030, 4, [0, 90], 0),                   # two-code lanes walking the feature axis in two tiles
])
def test_fused_equals_separate_and_oracle(bits, M, K, F, deg, seg, hubs):
    ops, plan, rowptr, col, val, x, seg_t, P, q, params = _setup(M, K, F, deg, bits, seg, seed=M + F + bits, hubs=hubs)
    init = torch.randn(M, F, generator=torch.Generator().manual_seed(1))
    vald = torch.from_numpy(val).cuda()
    # separate GPU path
    recv = torch.empty(K, F, device="cuda")
    ops.dequantize_tensor_for_all_procs(q, recv, params, seg_t, P, bits)
    out_sep = init.clone().cuda()
    plan.run(vald, recv, out_sep, accumulate=True)
    # fused
    out_fused = init.clone().cuda()
    ops.spmm_dequantized(None, None, vald, q, params, seg_t, P, bits, out_fused, plan=plan)
    torch.cuda.synchronize()
    assert torch.equal(out_fused, out_sep), "fused must equal dequantize-then-SpMM bit for bit"
    # oracle chain on the CPU
    q_ref, p_ref = orc.quant_rows(x.numpy(), seg, bits)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    d_ref = orc.dequant_rows(q_ref, p_ref, seg, bits, F)
    want = init.numpy().copy()
    orc.spmm_accumulate(rowptr, col, val, d_ref, want)
    got = out_fused.cpu().numpy()
    tol = 1e-6 + 1e-5 * np.abs(want)
    bad = np.abs(got - want) > tol
    if bad.any():  # long rows: adjudicate with the fp64 forward error bound
        f64 = orc.spmm_f64(rowptr, col, val, d_ref, init.numpy())
        S = orc.spmm_f64(rowptr, col, np.abs(val), np.abs(d_ref), np.abs(init.numpy()))
        bound = (np.diff(rowptr)[:, None] + 1.0) * 2.0 ** -24 * S
        bad &= np.abs(got - f64) > bound + 1e-6
    assert not bad.any()
    # overwrite mode and unit weights
    out_o = torch.full((M, F), 9.0, device="cuda")
    ops.spmm_dequantized(None, None, None, q, params, seg_t, P, bits, out_o, plan=plan, accumulate=False)
    out_o2 = torch.full((M, F), 9.0, device="cuda")
    plan.run(None, recv, out_o2, accumulate=False)
    assert torch.equal(out_o, out_o2)


def test_pre_post_aggregation_flow():
    # local rows [0, K_local) are fp32; remote boundary rows arrive int2-packed in 8 segments
    from super_gnn_amd import SparseTensor, SPMM_forward, SPMM_forward_quantized, synth
    from super_gnn_amd.quantizer import Quantizer_for_all_procs
    M, K_local, K_remote, F, bits = 20000, 20000, 5000, 128, 2
    rp_l, col_l = synth.rmat_graph(M, 150000, seed=6)
    rowptr_r, col_r, val_r = random_csr(M, K_remote, 4, seed=8, empty_frac=0.3, hubs=3, hub_deg=900)
    g = torch.Generator().manual_seed(7)
    x_local = torch.randn(K_local, F, generator=g)
    x_remote = torch.randn(K_remote, F, generator=g)
    wr = torch.tensor([0, 625, 1250, 1875, 2500, 3125, 3750, 4375, 5000], dtype=torch.int32)
    qz = Quantizer_for_all_procs(8, bits)
    npk = sum(qz.get_quantized_splits(625) for _ in range(8))
    q = torch.zeros(npk, F, dtype=torch.uint8, device="cuda")
    params = torch.zeros(K_remote, 2, device="cuda")
    qz.quantize_fp32_to_intX(x_remote.cuda(), q, params, wr)
    A_local = SparseTensor(rowptr=rp_l, col=col_l.to(torch.int64), value=torch.ones(col_l.numel()), sparse_sizes=(M, K_local), is_sorted=True).cuda()
    A_remote = SparseTensor(rowptr=torch.from_numpy(rowptr_r), col=torch.from_numpy(col_r), value=torch.from_numpy(val_r),
                            sparse_sizes=(M, K_remote), is_sorted=True).cuda()
    # (A) the reference's sequence: local SpMM, dequantize into recv_buf, remote SpMM onto the same out
    out_a = torch.zeros(M, F, device="cuda")
    SPMM_forward(A_local, x_local.cuda(), out_a)
    recv = torch.empty(K_remote, F, device="cuda")
    qz.dequantize_intX_to_fp32(q, recv, params, wr)
    SPMM_forward(A_remote, recv, out_a)
    # (B) fused
    out_b = torch.zeros(M, F, device="cuda")
    SPMM_forward(A_local, x_local.cuda(), out_b)
    SPMM_forward_quantized(A_remote, q, params, wr, bits, out_b)
    assert torch.equal(out_a, out_b)
    # and against the CPU oracle
    want = np.zeros((M, F), np.float32)
    orc.spmm_accumulate(rp_l.numpy(), col_l.numpy().astype(np.int64), np.ones(col_l.numel(), np.float32), x_local.numpy(), want)
    q_ref, p_ref = orc.quant_rows(x_remote.numpy(), wr.numpy(), bits)
    orc.spmm_accumulate(rowptr_r, col_r, val_r, orc.dequant_rows(q_ref, p_ref, wr.numpy(), bits, F), want)
    got = out_b.cpu().numpy()
    # one fp64 reference for the two-step sum: local part first, remote part accumulated onto it
    ones = np.ones(col_l.numel(), np.float32)
    cl = col_l.numpy().astype(np.int64)
    d_ref = orc.dequant_rows(q_ref, p_ref, wr.numpy(), bits, F)
    f64 = orc.spmm_f64(rp_l.numpy(), cl, ones, x_local.numpy()) + orc.spmm_f64(rowptr_r, col_r, val_r, d_ref)
    S = abs_sum64(rp_l.numpy(), cl, ones, x_local.numpy()) + abs_sum64(rowptr_r, col_r, val_r, d_ref)
    deg = np.diff(rp_l.numpy()) + np.diff(rowptr_r)
    assert_spmm_close(got, want, f64, S, deg, what="pre/post flow")


def test_fused_errors():
    ops, plan, rowptr, col, val, x, seg_t, P, q, params = _setup(50, 40, 64, 3, 2, [0, 40], seed=3)
    out = torch.zeros(50, 64, device="cuda")
    with pytest.raises(ValueError):
        ops.spmm_dequantized(None, None, None, q, params, seg_t, P, 3, out, plan=plan)
    with pytest.raises(ValueError):
        ops.spmm_dequantized(None, None, None, q, params, torch.tensor([0, 39], dtype=torch.int32), 1, 2, out, plan=plan)
    with pytest.raises(ValueError):
        ops.spmm_dequantized(None, None, None, q, params, seg_t, P, 2, torch.zeros(50, 63, device="cuda"), plan=plan)  # odd width


@pytest.mark.parametrize("bits", [8, 2])
@pytest.mark.parametrize("hubs", [0, 6])
def test_fused_with_bf16_params_equals_widened_params(bits, hubs):
    """params handed over as bf16 pairs == the same pairs widened to fp32 first (bitwise)."""
    M, K, F = 3000, 2000, 128
    seg = [0, 513, 1200, K]
    ops, plan, rowptr, col, val, x, seg_t, P, q, params = _setup(M, K, F, 9, bits, seg, seed=31 + bits, hubs=hubs)
    p16 = params.to(torch.bfloat16)
    v = torch.from_numpy(val).cuda()
    segs = ops.quant_segments(seg_t, bits)
    a = torch.randn(M, F, generator=torch.Generator().manual_seed(1)).cuda()
    b = a.clone()
    plan.run_quantized(v, q, p16, segs, bits, a, accumulate=True)
    plan.run_quantized(v, q, p16.to(torch.float32), segs, bits, b, accumulate=True)
    assert torch.equal(a, b)
    with pytest.raises(TypeError):
        plan.run_quantized(v, q, params.to(torch.float16), segs, bits, a, accumulate=True)


def test_fused_output_window_through_the_c_abi():
    # out as a 16-byte-aligned column window of a wider matrix (ldo > F): same bits, nothing else written;
    # a window that is not 16-byte aligned is refused
    from super_gnn_amd._lib import lib, check
    bits, F = 4, 128
    ops, plan, rowptr, col, val, x, seg_t, P, q, params = _setup(1500, 2000, F, 7, bits, [0, 700, 1303, 2000], seed=31, hubs=2)
    w = torch.from_numpy(val).cuda()
    segs = ops.quant_segments(seg_t, bits)
    ow = torch.randn(1500, F + 32, generator=torch.Generator().manual_seed(32)).cuda()
    want = ow[:, 16:16 + F].contiguous()
    plan.run_quantized(w, q, params, segs, bits, want, accumulate=True)
    got = ow.clone()
    slots = segs.row_slots(bits)
    stream = torch.cuda.current_stream().cuda_stream
    check(lib.sgnn_spmm_csr_dq_f32(plan._h, w.data_ptr(), q.data_ptr(), params.data_ptr(),
                                   slots.data_ptr() if slots is not None else None, bits, got.data_ptr() + 64, F, F + 32, 1,
                                   None, stream))
    torch.cuda.synchronize()
    assert torch.equal(got[:, 16:16 + F], want)
    assert torch.equal(got[:, :16], ow[:, :16]) and torch.equal(got[:, 16 + F:], ow[:, 16 + F:])
    rc = lib.sgnn_spmm_csr_dq_f32(plan._h, w.data_ptr(), q.data_ptr(), params.data_ptr(),
                                  slots.data_ptr() if slots is not None else None, bits, got.data_ptr() + 8, F, F + 32, 1,
                                  None, stream)
    assert rc != 0 and b"aligned" in lib.sgnn_last_error()


@pytest.fixture(scope="module")
def full_size_partition():
    # One partition at the largest configured size: 8 M local rows with ~320 M local edges, plus ~80 M edges
    # to 2 M remote boundary rows.  Built once on the GPU, together with the exact local product in fp64.
    import super_gnn_amd  # noqa: F401
    from super_gnn_amd import supergnn_ops as ops, synth
    dev = torch.device("cuda:0")
    Ml, Kr, F = 8_000_000, 2_000_000, 128
    rp_l, col_l = synth.rmat_graph(Ml, 160_000_000, seed=6, device=dev)
    g = torch.Generator(device=dev); g.manual_seed(7)
    deg_l = rp_l[1:] - rp_l[:-1]
    rows_r = torch.multinomial(deg_l.float() + 0.05, 80_000_000, replacement=True, generator=g)
    cols_r = torch.randint(0, Kr, (80_000_000,), generator=g, device=dev)
    rp_r, col_r = synth.csr_from_pairs(rows_r, cols_r, Ml, Kr, dedupe=True)
    del rows_r, cols_r
    x_l = torch.randint(-4, 5, (Ml, F), generator=g, device=dev).float()
    plan_l = ops.SpmmPlan(rp_l, col_l.to(torch.int32), Ml)
    plan_r = ops.SpmmPlan(rp_r, col_r.to(torch.int32), Kr)
    local = torch.zeros(Ml, F, dtype=torch.float64, device=dev)
    _index_add_product(local, rp_l, col_l, x_l)
    yield dict(ops=ops, dev=dev, Ml=Ml, Kr=Kr, F=F, g=g, x_l=x_l, plan_l=plan_l, plan_r=plan_r, rp_r=rp_r, col_r=col_r,
               local=local, max_deg_l=int(deg_l.max()), max_deg_r=int((rp_r[1:] - rp_r[:-1]).max()))


def _index_add_product(acc, rp, col, x, step=1 << 22):
    rows = torch.repeat_interleave(torch.arange(rp.numel() - 1, device=col.device), rp[1:] - rp[:-1])
    for e0 in range(0, int(col.numel()), step):
        e1 = min(int(col.numel()), e0 + step)
        acc.index_add_(0, rows[e0:e1], x[col[e0:e1]].double())


@pytest.mark.parametrize("bits", [2, 4])
def test_full_size_partition_exact_on_small_integers(bits, full_size_partition):
    # The remote rows arrive packed from 8 senders (ragged segments).  Integer features that the quantizer
    # represents exactly (every row spans exactly 2^bits - 1 steps of 1.0) and unit weights make every sum
    # exact in fp32, so local SpMM + fused remote SpMM has one right answer, checked against fp64.
    w = full_size_partition
    ops, dev, Ml, Kr, F, g = w["ops"], w["dev"], w["Ml"], w["Kr"], w["F"], w["g"]
    P, top = 8, 2 ** bits - 1
    assert w["max_deg_l"] * 4 + w["max_deg_r"] * (top + 5) < 2 ** 24
    zp = torch.randint(-5, 6, (Kr, 1), generator=g, device=dev).float()
    x_r = torch.randint(0, top + 1, (Kr, F), generator=g, device=dev).float() + zp
    x_r[:, 0:1] = zp
    x_r[:, 1:2] = zp + top
    bounds = [0] + sorted(int(v) for v in torch.randint(1, Kr, (P - 1,), generator=g, device=dev).tolist()) + [Kr]
    wr = torch.tensor(bounds, dtype=torch.int32)   # ragged: segments do not end on packed-row boundaries
    epb = 8 // bits
    npk = sum((bounds[i + 1] - bounds[i] + epb - 1) // epb for i in range(P))
    q = torch.empty(npk, F, dtype=torch.uint8, device=dev)
    prm = torch.empty(Kr, 2, device=dev)
    ops.quantize_tensor_for_all_procs(x_r, q, prm, wr, P, bits)
    assert torch.equal(prm[:, 0:1], zp) and bool((prm[:, 1] == 1.0).all())
    back = torch.empty_like(x_r)
    ops.dequantize_tensor_for_all_procs(q, back, prm, wr, P, bits)
    assert torch.equal(back, x_r)
    del back

    out = torch.full((Ml, F), 3.0, device=dev)
    w["plan_l"].run(None, w["x_l"], out, accumulate=False)
    w["plan_r"].run_quantized(None, q, prm, ops.quant_segments(wr, bits), bits, out, accumulate=True)
    want = w["local"].clone()
    _index_add_product(want, w["rp_r"], w["col_r"], x_r)
    assert torch.equal(out.double(), want)
