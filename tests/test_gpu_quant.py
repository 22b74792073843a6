"""GPU parity of the quantize / pack / unpack / dequantize path through the C ABI.
Codes, packed bytes and per-row params must be BIT-EXACT against the CPU restatement; dequantized
floats within one rounding of code*scale (see _util.dequant_atol)."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from _util import dequant_atol

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
KA = json.load(open(os.path.join(HERE, "golden", "known_answers.json")))
RV = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))


def _ops():
    import super_gnn_amd  # noqa: F401
    from super_gnn_amd import supergnn_ops
    return supergnn_ops


def _quant_gpu(x, seg, bits):
    ops = _ops()
    seg_t = torch.tensor(np.asarray(seg), dtype=torch.int32)
    P = seg_t.numel() - 1
    n, F = x.shape
    npk = int(orc.packed_rows(seg, bits).sum())
    xd = torch.from_numpy(x).cuda()
    q = torch.full((npk, F), 0xAB, dtype=torch.uint8, device="cuda")
    params = torch.full((n, 2), -7.0, device="cuda")
    ops.quantize_tensor_for_all_procs(xd, q, params, seg_t, P, bits)
    d = torch.full((n, F), 123.0, device="cuda")
    ops.dequantize_tensor_for_all_procs(q, d, params, seg_t, P, bits)
    torch.cuda.synchronize()
    return q.cpu().numpy(), params.cpu().numpy(), d.cpu().numpy()


@pytest.mark.parametrize("name", ["rows_int2", "rows_int8_ties", "rows_int4_two_rows", "rows_int2_two_segments"])
def test_known_answers(name):
    c = KA[name]
    q, params, _ = _quant_gpu(np.array(c["x"], dtype=np.float32), c["seg"], c["bits"])
    assert q.tolist() == c["q"]
    assert np.array_equal(params, np.array(c["params"], dtype=np.float32))


@pytest.mark.parametrize("bits", [8, 4, 2])
@pytest.mark.parametrize("n,F", [(2000, 128), (1001, 256), (4333, 123), (515, 602), (333, 64), (77, 100), (130, 1024),
                                 (41, 1200), (9, 4), (63, 16), (50, 2050), (3, 1),
                                 # rows of at most 16 floats: four, two lanes or one lane per row
                                 (3001, 4), (1027, 8), (2049, 10), (777, 12), (1500, 16), (999, 6), (1001, 3), (513, 2),
                                 (2500, 1), (800, 5), (700, 13),
                                 # 5 ... 12 vectors per row: four lanes per row, two or four vectors per lane
                                 (1111, 20), (901, 24), (1203, 28), (777, 36), (650, 44), (1024, 48), (300, 52)])
def test_rows_bit_exact_vs_oracle(bits, n, F):
    g = torch.Generator().manual_seed(n * 31 + F + bits)
    x = torch.randn(n, F, generator=g)
    x[::10] *= 100.0  # outlier rows
    x = x.numpy()
    if n > 5:
        x[3] = 0.5                      # constant row: scale 0 -> 1
        x[4, : min(F, 3)] = 0.0         # exact zeros
    q_ref, p_ref = orc.quant_rows(x, [0, n], bits)
    q, params, d = _quant_gpu(x, [0, n], bits)
    assert np.array_equal(params.view(np.uint32), p_ref.view(np.uint32)), "params differ"
    assert np.array_equal(q, q_ref), "packed bytes differ"
    d_ref = orc.dequant_rows(q_ref, p_ref, [0, n], bits, F)
    assert np.all(np.abs(d - d_ref) <= dequant_atol(p_ref[:, 0], p_ref[:, 1], bits)[:, None])
    assert np.all(np.abs(d - x) <= p_ref[:, 1:2] * 0.5 + 4 * dequant_atol(p_ref[:, 0], p_ref[:, 1], bits)[:, None])  # round-trip bound


@pytest.mark.parametrize("bits", [8, 4, 2])
@pytest.mark.parametrize("F", [128, 123, 602, 4, 10, 16, 7, 1, 24, 40])
def test_many_segments_bit_exact(bits, F):
    # the reference script's layout check: 256 random segments (tests/test_quantization_ops.py:130-148)
    rng = np.random.default_rng(bits + F)
    n, P = 4333, 256
    x = rng.standard_normal((n, F), dtype=np.float32)
    cuts = np.sort(rng.integers(0, n, size=P - 1))
    seg = np.concatenate([[0], cuts, [n]]).astype(np.int32)
    q_ref, p_ref = orc.quant_rows(x, seg, bits)
    q, params, d = _quant_gpu(x, seg, bits)
    assert np.array_equal(params.view(np.uint32), p_ref.view(np.uint32))
    assert np.array_equal(q, q_ref)
    # for_all_procs(x, ranges) == cat_p quantize_tensor(x[range_p]) (tests/test_quantization_ops.py:214-228)
    ops = _ops()
    parts = []
    for p in range(P):
        xs = torch.from_numpy(np.ascontiguousarray(x[seg[p]:seg[p + 1]])).cuda()
        m = xs.shape[0]
        epb = 8 // bits
        qp = torch.zeros(((m + epb - 1) // epb) * F, dtype=torch.uint8, device="cuda")
        pp = torch.zeros(m, 2, device="cuda")
        ops.quantize_tensor(xs, qp, pp, bits)
        parts.append(qp.view(-1, F).cpu().numpy())
    assert np.array_equal(q, np.concatenate(parts, axis=0))
    d_ref = orc.dequant_rows(q_ref, p_ref, seg, bits, F)
    assert np.all(np.abs(d - d_ref) <= dequant_atol(p_ref[:, 0], p_ref[:, 1], bits)[:, None])


@pytest.mark.parametrize("bits", [8, 2])
@pytest.mark.parametrize("P", [2, 62, 63, 64, 65, 126, 127, 128, 700])
def test_segment_counts_around_the_table_lookup_blocks(bits, P):
    # a wavefront looks its segment up 63 table entries at a time: counts on both sides of every block edge, with
    # empty segments (repeated cut points) and segments shorter than a packed row
    rng = np.random.default_rng(P * 10 + bits)
    n, F = 2900, 64
    x = rng.standard_normal((n, F), dtype=np.float32)
    cuts = np.sort(rng.integers(0, n + 1, size=P - 1))
    cuts[: (P - 1) // 4] = cuts[(P - 1) // 4]      # a run of empty segments at the front
    seg = np.concatenate([[0], cuts, [n]]).astype(np.int32)
    q_ref, p_ref = orc.quant_rows(x, seg, bits)
    q, params, d = _quant_gpu(x, seg, bits)
    assert np.array_equal(params.view(np.uint32), p_ref.view(np.uint32))
    assert np.array_equal(q, q_ref)
    d_ref = orc.dequant_rows(q_ref, p_ref, seg, bits, F)
    assert np.all(np.abs(d - d_ref) <= dequant_atol(p_ref[:, 0], p_ref[:, 1], bits)[:, None])


@pytest.mark.parametrize("bits", [8, 4, 2])
def test_reference_x86_vectors(bits):
    x = RV[f"qrows{bits}_x"]
    q, params, d = _quant_gpu(x, [0, x.shape[0]], bits)
    assert np.array_equal(q, RV[f"qrows{bits}_q"].reshape(-1, x.shape[1]))
    assert np.array_equal(params[:, 0], RV[f"qrows{bits}_min"]) and np.array_equal(params[:, 1], RV[f"qrows{bits}_scale"])
    assert np.all(np.abs(d - RV[f"qrows{bits}_deq"]) <= dequant_atol(params[:, 0], params[:, 1], bits)[:, None])


@pytest.mark.parametrize("F", [128, 37, 1500])
def test_nan_and_infinite_rows_vs_oracle(F):
    # the reference's strict compares make a NaN sticky only as element 0 (quantization_arm.cpp:98-101);
    # infinities give an infinite or NaN scale.  Whatever bytes and params the CPU arithmetic produces for
    # such rows, the kernels must produce the same ones (NaN params compared as NaN, payload aside).
    rng = np.random.default_rng(F)
    x = rng.standard_normal((12, F), dtype=np.float32)
    x[0, 0] = np.nan                       # NaN first: min = max = NaN
    x[1, F // 2] = np.nan                  # NaN later: ignored by the compares, its own code saturates to 0
    x[2, F - 1] = np.nan
    x[3, 1] = np.inf                       # max = +inf: scale = inf
    x[4, 2] = -np.inf                      # min = -inf: zero_point = -inf, scale = inf
    x[5, 0] = np.inf; x[5, 1] = -np.inf    # both
    x[6, 0] = -np.inf
    x[7, :] = np.inf                       # constant infinite row: inf - inf = NaN scale
    x[8, 0] = np.nan; x[8, 1] = np.inf
    x[9, :] = 3.0e38; x[9, 0] = -3.0e38    # finite extremes whose difference overflows to inf
    for bits in (8, 4, 2):
        q_ref, p_ref = orc.quant_rows(x, [0, 12], bits)
        q, params, _ = _quant_gpu(x, [0, 12], bits)
        nan_ref = np.isnan(p_ref)
        assert np.array_equal(np.isnan(params), nan_ref), bits
        assert np.array_equal(params[~nan_ref].view(np.uint32), p_ref[~nan_ref].view(np.uint32)), bits
        assert np.array_equal(q, q_ref), bits


def test_zero_signs_ties_denormals():
    ulp = np.float32(2.0 ** -149)
    x = np.array([[0.0, -0.0, 1.0, 2.0], [-0.0, 0.0, 1.0, 2.0], [3.0, 3.0, 3.0, 3.0], [-0.0, -0.0, -0.0, -0.0],
                  [-1.0, -0.0, 0.0, -2.0], [0.0, 3 * ulp, 6 * ulp, 9 * ulp], [0.5, 1.5, 2.5, 255.0],
                  [-2.0, -1.0, -0.0, 0.0], [-2.0, -1.0, 0.0, -0.0]], dtype=np.float32)
    x[6, 0] = 0.0
    for bits in (8, 4, 2):
        q_ref, p_ref = orc.quant_rows(x, [0, x.shape[0]], bits)
        q, params, _ = _quant_gpu(x, [0, x.shape[0]], bits)
        assert np.array_equal(params.view(np.uint32), p_ref.view(np.uint32)), bits
        assert np.array_equal(q, q_ref), bits
    # wide rows go through the two-pass kernel: same rule
    xw = np.zeros((5, 1500), dtype=np.float32)
    xw[0, 700] = -0.0; xw[0, 10] = 5.0
    xw[1, 0] = -0.0; xw[1, 1499] = -3.0
    xw[2, :] = -0.0; xw[2, 1400] = 0.0
    xw[3, :] = 2.0
    xw[4] = np.linspace(-1, 1, 1500, dtype=np.float32)
    for bits in (8, 2):
        q_ref, p_ref = orc.quant_rows(xw, [0, 5], bits)
        q, params, _ = _quant_gpu(xw, [0, 5], bits)
        assert np.array_equal(params.view(np.uint32), p_ref.view(np.uint32))
        assert np.array_equal(q, q_ref)


def test_v1_golden_and_oracle():
    ops = _ops()
    from super_gnn_amd.quantizer import QuantizerForMixedBits
    c = KA["v1_quantize"]  # the reference's own literals (tests/test_quantizer.py:57-84), CPU tensors in
    x = torch.tensor(c["x"], dtype=torch.float32)
    bits = torch.tensor(c["bits"])
    params = torch.empty(5, 3); params[:, 0] = bits
    rng = QuantizerForMixedBits.get_quantized_nodes_feat_range(5, 3, bits)
    q = torch.empty(int(rng[-1]), dtype=torch.uint8)
    QuantizerForMixedBits.quantize_fp32_to_intX(x, q, rng, params)
    assert rng.tolist() == c["range"] and q.tolist() == c["q"]
    assert torch.allclose(params[:, 1], x.min(dim=1)[0])
    assert torch.allclose(params[:, 2], (x.max(dim=1)[0] - params[:, 1]) / (2 ** params[:, 0] - 1))
    d = torch.empty(5, 3)
    QuantizerForMixedBits.dequantize_intX_to_fp32(q, d, rng, params)
    assert torch.all((d - x).abs() <= params[:, 2:3] * 0.5 * (1 + 1e-3) + 1e-6)
    # random mixed widths, odd F, against the oracle and the reference's x86 vectors
    for (xx, bb) in [(RV["v1_x"], RV["v1_bits"]),
                     (np.random.default_rng(0).standard_normal((300, 123), dtype=np.float32), np.random.default_rng(1).choice([8, 4, 2], 300))]:
        q_ref, rng_ref, p_ref = orc.quant_v1(xx, bb)
        pg = torch.zeros(xx.shape[0], 3, device="cuda"); pg[:, 0] = torch.from_numpy(bb.astype(np.float32)).cuda()
        qg = torch.zeros(int(rng_ref[-1]), dtype=torch.uint8, device="cuda")
        ops.quantize_tensor_v1(torch.from_numpy(xx).cuda(), qg, torch.from_numpy(rng_ref).cuda(), pg)
        assert np.array_equal(qg.cpu().numpy(), q_ref)
        assert np.array_equal(pg.cpu().numpy().view(np.uint32), p_ref.view(np.uint32))
        dg = torch.zeros(xx.shape, device="cuda")
        ops.dequantize_tensor_v1(qg, dg, torch.from_numpy(rng_ref).cuda(), pg)
        d_ref = orc.dequant_v1(q_ref, rng_ref, p_ref, xx.shape[1])
        assert np.all(np.abs(dg.cpu().numpy() - d_ref) <= dequant_atol(p_ref[:, 1], p_ref[:, 2], p_ref[:, 0])[:, None])
    # the bytes the reference's own x86 extension wrote for the first input (committed vectors)
    xx, bb = RV["v1_x"], RV["v1_bits"]
    pg = torch.zeros(xx.shape[0], 3, device="cuda"); pg[:, 0] = torch.from_numpy(bb.astype(np.float32)).cuda()
    qg = torch.zeros(int(RV["v1_range"][-1]), dtype=torch.uint8, device="cuda")
    ops.quantize_tensor_v1(torch.from_numpy(xx).cuda(), qg, torch.from_numpy(RV["v1_range"]).cuda(), pg)
    assert np.array_equal(qg.cpu().numpy(), RV["v1_q"])
    assert np.array_equal(pg.cpu().numpy(), RV["v1_params"])
    dg = torch.zeros(xx.shape, device="cuda")
    ops.dequantize_tensor_v1(qg, dg, torch.from_numpy(RV["v1_range"]).cuda(), pg)
    p_ref = RV["v1_params"]
    assert np.all(np.abs(dg.cpu().numpy() - RV["v1_deq"]) <= dequant_atol(p_ref[:, 1], p_ref[:, 2], p_ref[:, 0])[:, None])


def test_facades_and_errors():
    ops = _ops()
    from super_gnn_amd.quantizer import QuantizerForPureBits, Quantizer_for_all_procs
    x = torch.randn(37, 64, generator=torch.Generator().manual_seed(0))
    for bits in (8, 4, 2):
        size = QuantizerForPureBits.get_quantized_buffer_size(37, bits, 64)
        q = torch.zeros(size, dtype=torch.uint8); p = torch.zeros(37, 2)
        QuantizerForPureBits.quantize_fp32_to_intX(x, q, p, bits)  # CPU tensors: staged
        q_ref, p_ref = orc.quant_rows(x.numpy(), [0, 37], bits)
        assert np.array_equal(q.numpy().reshape(q_ref.shape), q_ref) and np.array_equal(p.numpy(), p_ref)
        d = torch.zeros(37, 64)
        QuantizerForPureBits.dequantize_intX_to_fp32(q, d, p, bits)
        assert torch.all((d - x).abs() <= p[:, 1:2] * 0.5 * (1 + 1e-5) + 1e-6)
    qz = Quantizer_for_all_procs(3, 2)
    wr = torch.tensor([0, 10, 10, 37], dtype=torch.int32)
    npk = sum(qz.get_quantized_splits(int(wr[i + 1] - wr[i])) for i in range(3))
    q = torch.zeros(npk, 64, dtype=torch.uint8, device="cuda"); p = torch.zeros(37, 2, device="cuda")
    qz.quantize_fp32_to_intX(x.cuda(), q, p, wr)
    q_ref, p_ref = orc.quant_rows(x.numpy(), wr.numpy(), 2)
    assert np.array_equal(q.cpu().numpy(), q_ref) and np.array_equal(p.cpu().numpy(), p_ref)
    with pytest.raises(ValueError):
        ops.quantize_tensor(x.cuda(), q, p, 3)
    with pytest.raises(ValueError):
        ops.quantize_tensor(x.cuda(), torch.zeros(5, dtype=torch.uint8, device="cuda"), p, 8)
    with pytest.raises(TypeError):
        ops.quantize_tensor(x.double().cuda(), q, p, 8)
    # zero rows: nothing to do, nothing written
    ops.quantize_tensor(torch.zeros(0, 64, device="cuda"), torch.zeros(0, dtype=torch.uint8, device="cuda"),
                        torch.zeros(0, 2, device="cuda"), 2)


@pytest.mark.parametrize("n,F", [(1_000_000, 256), (2_000_000, 128), (4_000_000, 64), (2_560_000, 100), (425_000, 602)])
@pytest.mark.parametrize("bits", [8, 4, 2])
def test_full_size_properties(bits, n, F):
    # the sweep's full shape (1M x 256, 10% outlier rows) and the same bytes as rows of 128 and 64 floats (the
    # widths the layers exchange; they take the eight-lanes-per-row kernel), ogbn-products' 100 floats (the quantizer
    # that walks runs of rows) and reddit's 602 (rows on 8-byte boundaries): size-independent properties plus an
    # exact comparison of every row with the oracle
    from super_gnn_amd import synth
    ops = _ops()
    x = synth.boundary_features(n, F, seed=5, device="cuda")
    epb = 8 // bits
    seg = torch.tensor([0, n], dtype=torch.int32)
    q = torch.empty((n + epb - 1) // epb, F, dtype=torch.uint8, device="cuda")
    p = torch.empty(n, 2, device="cuda")
    ops.quantize_tensor_for_all_procs(x, q, p, seg, 1, bits)
    d = torch.empty(n, F, device="cuda")
    ops.dequantize_tensor_for_all_procs(q, d, p, seg, 1, bits)
    mn, mx = x.min(dim=1).values, x.max(dim=1).values
    assert torch.equal(p[:, 0], mn)
    # divide by a TENSOR: torch turns division by a Python scalar into a multiply by its reciprocal on the GPU
    assert torch.equal(p[:, 1], (mx - mn) / torch.full_like(mx, float(2 ** bits - 1)))
    # half a step, plus fp32 rounding of x - zp and of code*scale + zp at the magnitude of the row
    slack = (p[:, 0:1].abs() + float(2 ** bits - 1) * p[:, 1:2]) * 2.0 ** -22 + 1e-30
    assert bool(((d - x).abs() <= p[:, 1:2] * 0.5 + slack).all())
    assert torch.equal(d.min(dim=1).values, mn)
    # idempotence: quantizing the dequantized rows reproduces the same bytes
    q2 = torch.empty_like(q); p2 = torch.empty_like(p)
    ops.quantize_tensor_for_all_procs(d, q2, p2, seg, 1, bits)
    assert float((q2 != q).float().mean()) < 1e-3  # scale is re-derived from rounded extremes; codes agree almost everywhere
    # every one of the 1 M rows against the oracle: packed bytes and params bit for bit, floats within one
    # rounding of code*scale
    xh = x.cpu().numpy()
    q_ref, p_ref = orc.quant_rows(xh, [0, n], bits)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    assert np.array_equal(p.cpu().numpy().view(np.uint32), p_ref.view(np.uint32))
    d_ref = orc.dequant_rows(q_ref, p_ref, [0, n], bits, F)
    assert np.all(np.abs(d.cpu().numpy() - d_ref) <= dequant_atol(p_ref[:, 0], p_ref[:, 1], bits)[:, None])


@pytest.mark.parametrize("F", [256, 128, 64, 602, 123, 100])
@pytest.mark.parametrize("bits", [8, 4, 2])
def test_fast_quotient_equals_ieee_division(bits, F):
    """The kernel forms (x-zp)*RN(1/scale) and falls back to the IEEE division near half-integers;
    its bytes must equal those of the all-IEEE variant (SGNN_QUANT_EXACT_DIV=1) on the full-size
    input and on rows built to sit on rounding ties."""
    import os
    from super_gnn_amd import synth
    ops = _ops()
    qmax = (1 << bits) - 1
    g = torch.Generator(device="cuda"); g.manual_seed(bits)
    # (F = 602 / 123: the rows start on 8- / 4-byte boundaries and the default kernel reads them with unaligned
    # 16-byte loads, while the all-IEEE variant is the lane-group kernel with float2 / scalar lanes)
    n = (256_000_000 if F % 4 == 0 else 64_000_000) // F
    x = synth.boundary_features(n, F, seed=5, device="cuda")
    # adversarial block: min 0, max qmax*s, values at (k + 0.5 +- tiny) * s for assorted scales s
    na = 4096
    s = torch.rand(na, 1, generator=g, device="cuda") * 3 + 0.01
    k = torch.randint(0, qmax, (na, F), generator=g, device="cuda").float()
    # quotients a few ulps either side of the tie, and -- for the narrower guard bands of int4 / int2 -- up to
    # and beyond the edge of the band (2^-13, 2^-17, 2^-19 absolute)
    eps = (torch.randint(-3, 4, (na, F), generator=g, device="cuda").float()) * 2.0 ** -22
    eps[na // 2:] *= 2.0 ** torch.randint(0, 8, (na - na // 2, F), generator=g, device="cuda").float()
    adv = (k + 0.5) * (1 + eps) * s
    adv[:, 0] = 0.0
    adv[:, 1] = qmax * s[:, 0]
    x[:na] = adv
    # rows with extreme scales: reciprocal not a normal number -> whole-row fallback
    x[na] = torch.linspace(0, 1e-38, F, device="cuda")
    x[na + 1] = torch.linspace(-3e38, 3e38, F, device="cuda")
    epb = 8 // bits
    seg = torch.tensor([0, n], dtype=torch.int32)
    outs = []
    for exact in ("0", "1"):
        os.environ["SGNN_QUANT_EXACT_DIV"] = exact
        q = torch.empty((n + epb - 1) // epb, F, dtype=torch.uint8, device="cuda")
        p = torch.empty(n, 2, device="cuda")
        ops.quantize_tensor_for_all_procs(x, q, p, seg, 1, bits)
        torch.cuda.synchronize()
        outs.append((q, p))
    os.environ.pop("SGNN_QUANT_EXACT_DIV")
    assert torch.equal(outs[0][0], outs[1][0])
    assert torch.equal(outs[0][1].view(torch.int32), outs[1][1].view(torch.int32))
    xs = x[: na + 8].cpu().numpy()
    q_ref, p_ref = orc.quant_rows(xs, [0, na + 8], bits)
    assert np.array_equal(outs[0][0][: (na + 8) // epb].cpu().numpy(), q_ref)


# ------------------------------------------------------------------------------------------------
# wire-side variants: gathered input rows, bf16 (zero_point, scale)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("bits", [8, 4, 2])
@pytest.mark.parametrize("F", [128, 256, 100, 37, 1200, 602])
def test_gathering_quantizer_equals_index_select_then_quantize(bits, F):
    from super_gnn_amd import supergnn_ops as ops
    gen = torch.Generator().manual_seed(bits * 1000 + F)
    src = torch.randn(5000, F, generator=gen).cuda()
    idx = torch.randint(0, 5000, (3001,), generator=gen).cuda()
    wr = torch.tensor([0, 700, 700, 1999, 3001], dtype=torch.int32)
    npk = sum(-(-int(b - a) // (8 // bits)) for a, b in zip(wr[:-1], wr[1:]))
    q_a = torch.zeros((npk, F), dtype=torch.uint8, device="cuda"); p_a = torch.zeros((3001, 2), device="cuda")
    q_b = torch.zeros_like(q_a); p_b = torch.zeros_like(p_a)
    ops.quantize_tensor_for_all_procs(src[idx].contiguous(), q_a, p_a, wr, 4, bits)
    ops.quantize_tensor_for_all_procs(src, q_b, p_b, wr, 4, bits, row_index=idx)
    assert torch.equal(q_a, q_b) and torch.equal(p_a, p_b)
    # strided source (a column window of a wider matrix)
    wide = torch.randn(5000, F + 8, generator=gen).cuda()
    view = wide[:, 4:4 + F]
    q_c = torch.zeros_like(q_a); p_c = torch.zeros_like(p_a)
    ops.quantize_tensor_for_all_procs(view, q_c, p_c, wr, 4, bits, row_index=idx)
    ops.quantize_tensor_for_all_procs(view[idx].contiguous(), q_a, p_a, wr, 4, bits)
    assert torch.equal(q_a, q_c) and torch.equal(p_a, p_c)
    # a window whose rows start on odd 4-byte boundaries (odd leading dimension, odd column offset)
    wide = torch.randn(5000, F + 7, generator=gen).cuda()
    view = wide[:, 3:3 + F]
    ops.quantize_tensor_for_all_procs(view, q_c, p_c, wr, 4, bits, row_index=idx)
    ops.quantize_tensor_for_all_procs(view[idx].contiguous(), q_a, p_a, wr, 4, bits)
    assert torch.equal(q_a, q_c) and torch.equal(p_a, p_c)
    with pytest.raises(IndexError):
        ops.quantize_tensor_for_all_procs(src, q_b, p_b, wr, 4, bits, row_index=idx + 4000)


@pytest.mark.parametrize("bits", [8, 4, 2])
@pytest.mark.parametrize("F", [128, 64, 602, 1200])
def test_bf16_params_equal_torch_casts(bits, F):
    """bf16 params out of the quantizer == torch's fp32->bf16 copy of the fp32 params (codes
    unchanged); dequantizing with bf16 params == dequantizing with their exact fp32 widening."""
    from super_gnn_amd import supergnn_ops as ops
    gen = torch.Generator().manual_seed(bits + F)
    n = 2049
    x = (torch.randn(n, F, generator=gen) * torch.logspace(-20, 20, n).unsqueeze(1)).cuda()
    x[5] = 0.0; x[6] = -0.0; x[7, 0] = float("nan"); x[8] = 3.0e38; x[8, 1] = -3.0e38
    wr = torch.tensor([0, 1000, n], dtype=torch.int32)
    npk = sum(-(-int(b - a) // (8 // bits)) for a, b in zip(wr[:-1], wr[1:]))
    q32 = torch.zeros((npk, F), dtype=torch.uint8, device="cuda"); p32 = torch.zeros((n, 2), device="cuda")
    q16 = torch.zeros_like(q32); p16 = torch.zeros((n, 2), dtype=torch.bfloat16, device="cuda")
    ops.quantize_tensor_for_all_procs(x, q32, p32, wr, 2, bits)
    ops.quantize_tensor_for_all_procs(x, q16, p16, wr, 2, bits)
    assert torch.equal(q32, q16)
    want16 = p32.to(torch.bfloat16)
    assert torch.equal(p16.view(torch.int16)[~want16.isnan()], want16.view(torch.int16)[~want16.isnan()])
    assert torch.equal(p16.isnan(), want16.isnan())
    a = torch.zeros((n, F), device="cuda"); b = torch.zeros((n, F), device="cuda")
    ops.dequantize_tensor_for_all_procs(q16, a, p16, wr, 2, bits)
    ops.dequantize_tensor_for_all_procs(q16, b, p16.to(torch.float32), wr, 2, bits)
    assert torch.equal(a.nan_to_num(1.5, 2.5, 3.5), b.nan_to_num(1.5, 2.5, 3.5))


@pytest.mark.parametrize("bits", [8, 4, 2])
@pytest.mark.parametrize("F", [4, 64, 100, 128, 256, 600, 1028, 2052, 602, 123, 6, 3, 1, 2050, 5, 301, 1433])
def test_flat_and_row_tiled_dequantizers_agree(bits, F, monkeypatch):
    """The flat-output kernels (default; at odd widths also the general one that the two-row kernel
    replaces) and the row-tiled kernels are decompositions of the same arithmetic: same bits out,
    ragged multi-segment tables included."""
    from super_gnn_amd import supergnn_ops as ops
    gen = torch.Generator().manual_seed(bits * 7 + F)
    n = 3001
    x = torch.randn(n, F, generator=gen).cuda()
    for wr in ([0, n], [0, 1, 2, 2, 777, 2998, n]):
        wr_t = torch.tensor(wr, dtype=torch.int32)
        P = len(wr) - 1
        npk = sum(-(-(b - a) // (8 // bits)) for a, b in zip(wr[:-1], wr[1:]))
        q = torch.zeros((npk, F), dtype=torch.uint8, device="cuda"); prm = torch.zeros((n, 2), device="cuda")
        ops.quantize_tensor_for_all_procs(x, q, prm, wr_t, P, bits)
        outs = []
        for flat, odd2 in (("1", "1"), ("0", "1"), ("1", "0")):
            monkeypatch.setenv("SGNN_DEQUANT_FLAT", flat)
            monkeypatch.setenv("SGNN_DEQUANT_ODD2", odd2)
            o = torch.full((n, F), 7.0, device="cuda")
            ops.dequantize_tensor_for_all_procs(q, o, prm, wr_t, P, bits)
            outs.append(o)
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


def test_cpu_runnable_configuration_int8_boundary_rows():
    """2 000 boundary rows x 128 N(0,1) features, int8, one segment: bytes and params bit-exact,
    dequantized floats within one rounding of code*scale."""
    from super_gnn_amd import QuantizerForPureBits
    x = torch.randn(2000, 128, generator=torch.Generator().manual_seed(0))
    seg = np.array([0, 2000], np.int32)
    q_ref, p_ref = orc.quant_rows(x.numpy(), seg, 8)
    q = torch.zeros(2000 * 128, dtype=torch.uint8, device="cuda"); p = torch.zeros(2000, 2, device="cuda")
    QuantizerForPureBits.quantize_fp32_to_intX(x.cuda(), q, p, 8)
    assert np.array_equal(q.cpu().numpy().reshape(2000, 128), q_ref) and np.array_equal(p.cpu().numpy(), p_ref)
    back = torch.zeros(2000, 128, device="cuda")
    QuantizerForPureBits.dequantize_intX_to_fp32(q, back, p, 8)
    want = orc.dequant_rows(q_ref, p_ref, seg, 8, 128)
    tol = dequant_atol(p_ref[:, 0], p_ref[:, 1], 8)[:, None]
    assert np.all(np.abs(back.cpu().numpy() - want) <= tol)
    assert np.all(np.abs(back.cpu().numpy() - x.numpy()) <= p_ref[:, 1:2] * 0.5 * (1 + 1e-6) + 4 * tol)


@pytest.mark.parametrize("F", [4, 12, 32, 36, 64, 100, 128, 132, 256, 260, 512, 600, 1024, 1028, 37])
def test_v1_mixed_bits_all_widths(F):
    """Feature-packed mixed-bit rows (2/4/8 bits chosen per row, so row byte offsets fall on every
    alignment): bytes and params bit-exact vs the oracle, floats within one rounding; widths on both
    the float4 kernels (F % 4 == 0, F <= 1024) and the general ones."""
    from super_gnn_amd import supergnn_ops as ops
    rng_ = np.random.default_rng(F)
    n = 777
    x = (rng_.standard_normal((n, F)) * np.exp(rng_.uniform(-5, 5, size=(n, 1)))).astype(np.float32)
    x[5] = 0.0; x[6] = -0.0; x[7] = 2.5
    if F > 1:
        x[8, 0] = 0.0; x[8, 1] = -0.0
    bits = rng_.choice([2, 4, 8], size=n)
    # rows of rounding ties and their one-ulp neighbours: min 0, max 2^b - 1 (scale exactly 1), and a
    # scale that is not a power of two
    for row, b in ((9, 8), (10, 4), (11, 2), (12, 8), (13, 2)):
        bits[row] = b
        qmax = float((1 << b) - 1)
        ties = (rng_.integers(0, int(qmax), size=F) + 0.5).astype(np.float32)
        ties = np.nextafter(ties, ties + rng_.choice([-1.0, 0.0, 1.0], size=F).astype(np.float32)).astype(np.float32)
        ties[0], ties[-1] = 0.0, qmax
        x[row] = ties * (np.float32(1.0) if row < 12 else np.float32(0.3))
    q_ref, r_ref, p_ref = orc.quant_v1(x, bits)
    q = torch.zeros(q_ref.shape[0], dtype=torch.uint8, device="cuda")
    prm = torch.zeros(n, 3, device="cuda"); prm[:, 0] = torch.from_numpy(bits.astype(np.float32)).cuda()
    r = torch.from_numpy(r_ref).cuda()
    ops.quantize_tensor_v1(torch.from_numpy(x).cuda(), q, r, prm)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    assert np.array_equal(prm.cpu().numpy(), p_ref)
    back = torch.full((n, F), 9.0, device="cuda")
    ops.dequantize_tensor_v1(q, back, r, prm)
    want = orc.dequant_v1(q_ref, r_ref, p_ref, F)
    tol = dequant_atol(p_ref[:, 1], p_ref[:, 2], bits)[:, None]
    assert np.all(np.abs(back.cpu().numpy() - want) <= tol)


@pytest.mark.parametrize("F", [32, 64, 128, 256, 512])
def test_v1_rows_with_gaps_and_illegal_widths(F):
    """The v1 quantizer gathers a wavefront's rows into one run of stores when the rows' byte ranges follow one
    another; ranges with gaps between rows, rows of an illegal bit width (left untouched, as the reference leaves
    them, quantization_x86.cpp:244-245) and the last, partly filled wavefront must take the per-row stores and
    leave every byte outside the rows' ranges alone."""
    from super_gnn_amd import supergnn_ops as ops, _lib
    rng_ = np.random.default_rng(100 + F)
    n = 1003
    x = rng_.standard_normal((n, F)).astype(np.float32)
    bits = rng_.choice([2, 4, 8], size=n)
    q_ref, r_ref, p_ref = orc.quant_v1(x, bits)
    length = np.diff(r_ref)
    for gaps, bad in ((True, []), (False, [17, 500, 501, 1002]), (True, [0, 64])):
        start = r_ref[:-1] + (3 * np.arange(n) if gaps else 0)
        rng_dev = np.concatenate([start, [start[-1] + length[-1] + (3 if gaps else 0)]]).astype(np.int64)
        total = int(rng_dev[-1]) + 8
        q = torch.full((total,), 0xAB, dtype=torch.uint8, device="cuda")
        prm = torch.full((n, 3), -7.0, device="cuda")
        b_dev = bits.astype(np.float32).copy()
        b_dev[bad] = 3.0
        prm[:, 0] = torch.from_numpy(b_dev).cuda()
        xd, rd = torch.from_numpy(x).cuda(), torch.from_numpy(rng_dev).cuda()
        # through the C ABI: the Python wrapper refuses illegal widths before the library sees them
        _lib.check(_lib.lib.sgnn_quant_v1_f32(xd.data_ptr(), q.data_ptr(), rd.data_ptr(), prm.data_ptr(), n, F, ops._stream()))
        got, gp = q.cpu().numpy(), prm.cpu().numpy()
        want = np.full(total, 0xAB, dtype=np.uint8)
        for i in range(n):
            if i in bad:
                assert gp[i, 1] == -7.0 and gp[i, 2] == -7.0
                continue
            want[start[i]:start[i] + length[i]] = q_ref[r_ref[i]:r_ref[i + 1]]
            assert gp[i, 1] == p_ref[i, 1] and gp[i, 2] == p_ref[i, 2]
        assert np.array_equal(got, want), f"gaps={gaps} bad={bad}"
        # and back: rows of an illegal width keep what the output held
        back = torch.full((n, F), 9.0, device="cuda")
        _lib.check(_lib.lib.sgnn_dequant_v1_f32(q.data_ptr(), back.data_ptr(), rd.data_ptr(), prm.data_ptr(), n, F, ops._stream()))
        wantx = orc.dequant_v1(q_ref, r_ref, p_ref, F)
        wantx[bad] = 9.0
        tol = dequant_atol(p_ref[:, 1], p_ref[:, 2], bits)[:, None]
        tol[bad] = 0.0
        assert np.all(np.abs(back.cpu().numpy() - wantx) <= tol)


@pytest.mark.parametrize("bits", [8, 4, 2])
@pytest.mark.parametrize("F", [602, 123, 100, 128])
def test_buffers_at_odd_addresses(bits, F):
    """fp32 rows that start 4 bytes into an allocation and packed bytes that start 1 or 2 bytes into theirs (views
    of larger buffers): every kernel choice must still write exactly the oracle's bytes, and only those."""
    ops = _ops()
    n = 1237
    rng_ = np.random.default_rng(bits * 10 + F)
    x = rng_.standard_normal((n, F)).astype(np.float32)
    seg = [0, 400, 401, n]
    q_ref, p_ref = orc.quant_rows(x, seg, bits)
    npk = q_ref.shape[0]
    for xoff, qoff in ((1, 1), (2, 2), (0, 3), (3, 0)):
        xb = torch.zeros(n * F + 8, device="cuda")
        xv = xb[xoff:xoff + n * F].view(n, F)
        xv.copy_(torch.from_numpy(x))
        qb = torch.full((npk * F + 8,), 0xCD, dtype=torch.uint8, device="cuda")
        qv = qb[qoff:qoff + npk * F].view(npk, F)
        prm = torch.zeros(n, 2, device="cuda")
        ops.quantize_tensor_for_all_procs(xv, qv, prm, torch.tensor(seg, dtype=torch.int32), 3, bits)
        got = qb.cpu().numpy()
        assert np.array_equal(got[qoff:qoff + npk * F].reshape(npk, F), q_ref), (xoff, qoff)
        assert (got[:qoff] == 0xCD).all() and (got[qoff + npk * F:] == 0xCD).all(), "bytes outside the packed rows were written"
        assert np.array_equal(prm.cpu().numpy().view(np.uint32), p_ref.view(np.uint32))
        ob = torch.full((n * F + 8,), 7.0, device="cuda")
        ov = ob[xoff:xoff + n * F].view(n, F)
        ops.dequantize_tensor_for_all_procs(qv, ov, prm, torch.tensor(seg, dtype=torch.int32), 3, bits)
        d_ref = orc.dequant_rows(q_ref, p_ref, seg, bits, F)
        o = ob.cpu().numpy()
        assert np.all(np.abs(o[xoff:xoff + n * F].reshape(n, F) - d_ref) <= dequant_atol(p_ref[:, 0], p_ref[:, 1], bits)[:, None])
        assert (o[:xoff] == 7.0).all() and (o[xoff + n * F:] == 7.0).all(), "floats outside the rows were written"


@pytest.mark.parametrize("n,F", [(9_000_000, 128), (11_000_000, 100), (9_000_000, 123)])
def test_offsets_beyond_four_gigabytes(n, F):
    # 9 M x 128 fp32 = 4.6 GB: byte offsets of the last rows do not fit 32 bits, and neither does the number of
    # ELEMENTS behind the first rows at F = 100 / 123 (the widths that take the quantizer which walks runs of rows,
    # the second one with rows that are not whole float4).  Params against torch's
    # min/max, the round-trip bound everywhere, and the last rows of every segment bit-exact against the oracle.
    ops = _ops()
    bits, P = 2, 3
    epb = 8 // bits
    g = torch.Generator(device="cuda"); g.manual_seed(41)
    x = torch.randn(n, F, generator=g, device="cuda")
    bounds = [0, 2_999_999, 6_000_002, n]
    seg = torch.tensor(bounds, dtype=torch.int32)
    pk = [(bounds[i + 1] - bounds[i] + epb - 1) // epb for i in range(P)]
    q = torch.empty(sum(pk), F, dtype=torch.uint8, device="cuda")
    p = torch.empty(n, 2, device="cuda")
    ops.quantize_tensor_for_all_procs(x, q, p, seg, P, bits)
    mn, mx = x.min(dim=1).values, x.max(dim=1).values
    assert torch.equal(p[:, 0], mn)
    assert torch.equal(p[:, 1], (mx - mn) / torch.full_like(mx, float(2 ** bits - 1)))
    d = torch.empty_like(x)
    ops.dequantize_tensor_for_all_procs(q, d, p, seg, P, bits)
    slack = (p[:, 0:1].abs() + float(2 ** bits - 1) * p[:, 1:2]) * 2.0 ** -22 + 1e-30
    assert bool(((d - x).abs() <= p[:, 1:2] * 0.5 + slack).all())
    pstart = 0
    for i in range(P):
        rows = bounds[i + 1] - bounds[i]
        tail = (rows - 1) // epb * epb - 4096          # a packed-row-aligned window ending at the segment's last row
        xs = x[bounds[i] + tail:bounds[i + 1]].cpu().numpy()
        q_ref, p_ref = orc.quant_rows(xs, [0, xs.shape[0]], bits)
        q_got = q[pstart + tail // epb:pstart + pk[i]].cpu().numpy()
        assert np.array_equal(q_got, q_ref)
        assert np.array_equal(p[bounds[i] + tail:bounds[i + 1]].cpu().numpy().view(np.uint32), p_ref.view(np.uint32))
        d_ref = orc.dequant_rows(q_ref, p_ref, [0, xs.shape[0]], bits, F)
        d_got = d[bounds[i] + tail:bounds[i + 1]].cpu().numpy()
        assert np.all(np.abs(d_got - d_ref) <= dequant_atol(p_ref[:, 0], p_ref[:, 1], bits)[:, None])
        pstart += pk[i]


def _special_rows(n, F, rng):
    """Random rows with the cases the per-row rules turn on: outliers, a constant row, NaN as element 0 and later,
    infinities, and rows whose minimum or maximum is a zero with zeros of both signs at random places."""
    x = rng.standard_normal((n, F)).astype(np.float32)
    x[::10] *= 100.0
    if n < 40:
        return x
    x[3] = 0.5
    x[5, 0] = np.nan
    x[6, F // 2] = np.nan
    x[7, F - 1] = np.inf
    x[8, 1] = -np.inf
    for r in range(12, 40):     # signed zeros: non-negative rows (min is a zero), non-positive rows (max is one), all-zero rows
        kind = r % 4
        row = np.abs(x[r]) if kind in (0, 1) else -np.abs(x[r]) if kind == 2 else np.zeros(F, np.float32)
        k = rng.integers(1, 6)
        pos = rng.choice(F, size=min(k, F), replace=False)
        row[pos] = np.where(rng.random(pos.size) < 0.5, np.float32(0.0), np.float32(-0.0))
        if kind == 3:
            row[:] = np.where(rng.random(F) < (0.5 if r % 8 == 3 else 0.02), np.float32(-0.0), np.float32(0.0))
        if r % 5 == 0:
            row[pos] = -0.0     # zeros of one sign only
        x[r] = row
    return x


@pytest.mark.parametrize("stream", ["0", "1"])
@pytest.mark.parametrize("bits", [8, 4, 2])
@pytest.mark.parametrize("F", [16, 20, 36, 100, 123, 128, 200, 301, 602, 1000, 1200, 1433])
def test_stream_and_lane_group_quantizers_write_the_oracles_bytes(stream, bits, F, monkeypatch):
    """SGNN_QUANT_STREAM forces (1) or forbids (0) the quantizer that walks a run of consecutive rows vector by
    vector; by default the library picks per width.  Either kernel must write exactly the oracle's bytes and
    params: ragged per-peer segments (short last groups, a chunk spanning two segments), special rows."""
    monkeypatch.setenv("SGNN_QUANT_STREAM", stream)
    rng = np.random.default_rng(1000 * bits + F)
    n = 997
    x = _special_rows(n, F, rng)
    for seg in ([0, n], [0, 1, 2, 7, 7, 130, 131, 555, n]):
        q_ref, p_ref = orc.quant_rows(x, seg, bits)
        q, params, d = _quant_gpu(x, seg, bits)
        nan_ref = np.isnan(p_ref)
        assert np.array_equal(np.isnan(params), nan_ref), seg
        assert np.array_equal(params[~nan_ref].view(np.uint32), p_ref[~nan_ref].view(np.uint32)), seg
        assert np.array_equal(q, q_ref), seg
    # the same rows picked out of a wider tensor by a row index (repeats, the tensor's last row at several places,
    # rows that start on odd 4-byte boundaries): the oracle on the gathered copy
    from super_gnn_amd import supergnn_ops as ops
    wide = np.zeros((n, F + 3), np.float32)
    wide[:, 1:1 + F] = x
    idx = rng.integers(0, n, size=613)
    idx[[0, 100, 611, 612]] = n - 1
    seg = [0, 5, 5, 300, 613]
    q_ref, p_ref = orc.quant_rows(np.ascontiguousarray(x[idx]), seg, bits)
    epb = 8 // bits
    npk = sum(-(-(b - a) // epb) for a, b in zip(seg[:-1], seg[1:]))
    view = torch.from_numpy(wide).cuda()[:, 1:1 + F]
    q = torch.zeros(npk, F, dtype=torch.uint8, device="cuda")
    params = torch.zeros(len(idx), 2, device="cuda")
    ops.quantize_tensor_for_all_procs(view, q, params, torch.tensor(seg, dtype=torch.int32), len(seg) - 1, bits,
                                      row_index=torch.from_numpy(idx).cuda())
    params = params.cpu().numpy()
    nan_ref = np.isnan(p_ref)
    assert np.array_equal(np.isnan(params), nan_ref)
    assert np.array_equal(params[~nan_ref].view(np.uint32), p_ref[~nan_ref].view(np.uint32))
    assert np.array_equal(q.cpu().numpy(), q_ref)
