"""Pins the CPU restatement of the quantize / pack / unpack / dequantize path WITHOUT a GPU:
hand-derived known answers, the reference's own golden literals, vectors produced by the
reference's x86 extension (tests/golden/ref_vectors.npz), the live extension when oracle/_ref is
built, an independent numpy formulation, and the reference's segment-concatenation invariant."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from _util import dequant_atol

HERE = os.path.dirname(os.path.abspath(__file__))
KA = json.load(open(os.path.join(HERE, "golden", "known_answers.json")))
RV = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))


@pytest.mark.parametrize("name", ["rows_int2", "rows_int8_ties", "rows_int4_two_rows", "rows_int2_two_segments"])
def test_rows_known_answers(name):
    c = KA[name]
    x = np.array(c["x"], dtype=np.float32)
    q, params = orc.quant_rows(x, c["seg"], c["bits"])
    assert q.tolist() == c["q"]
    assert np.array_equal(params, np.array(c["params"], dtype=np.float32))
    q2, params2 = orc.quant_rows_numpy(x, c["seg"], c["bits"])
    assert np.array_equal(q, q2) and np.array_equal(params, params2)


def test_v1_reference_golden_bytes():
    c = KA["v1_quantize"]  # literals of the reference's tests/test_quantizer.py:57-84
    x = np.array(c["x"], dtype=np.float32)
    q, rng, params = orc.quant_v1(x, c["bits"])
    assert q.tolist() == c["q"]
    assert rng.tolist() == c["range"]
    b = np.array(c["bits"], dtype=np.float32)
    assert np.allclose(params[:, 1], x.min(axis=1))
    assert np.allclose(params[:, 2], (x.max(axis=1) - x.min(axis=1)) / (2 ** b - 1))


def test_v1_reference_golden_dequant():
    c = KA["v1_dequantize"]  # tests/test_quantizer.py:87-114
    params = np.array(c["params"], dtype=np.float32)
    rng = orc.v1_range(params[:, 0].astype(np.int64), 3)
    x = orc.dequant_v1(np.array(c["q"], dtype=np.uint8), rng, params, 3)
    # The reference asserts default-tolerance allclose against the ORIGINAL floats, which its own
    # arithmetic cannot meet (byte 7 at 4 bits is code 7 -> 0.4 + 7*0.013333 = 0.4933, not 0.5).
    # What the literals do pin: every value is the original to within half a quantization step.
    want = np.array(c["x"], dtype=np.float32)
    assert np.all(np.abs(x - want) <= params[:, 2:3] * 0.5 * (1 + 1e-3) + 1e-6)
    assert np.allclose(x[0], [0.1 + 127 * 7.8431e-04, 0.1, 0.1 + 255 * 7.8431e-04], rtol=1e-6)
    assert np.allclose(x[1], [0.4, 0.4 + 7 * 1.3333e-02, 0.4 + 15 * 1.3333e-02], rtol=1e-6)


def test_v1_range_closed_forms():
    for c in KA["v1_range"]:  # tests/test_quantizer.py:29-55
        assert orc.v1_range(c["bits"], c["feat_len"]).tolist() == c["range"]


@pytest.mark.parametrize("bits", [8, 4, 2])
def test_rows_vs_reference_x86_vectors(bits):
    x, mn, sc = RV[f"qrows{bits}_x"], RV[f"qrows{bits}_min"], RV[f"qrows{bits}_scale"]
    q_ref = RV[f"qrows{bits}_q"].reshape(-1, x.shape[1])
    # packing + rounding with the caller-supplied params the x86 build takes
    assert np.array_equal(orc.quant_rows_given_params(x, mn, sc, bits), q_ref)
    # and our own per-row params reproduce the same min/scale, hence the same bytes
    q, params = orc.quant_rows(x, [0, x.shape[0]], bits)
    assert np.array_equal(params[:, 0], mn) and np.array_equal(params[:, 1], sc)
    assert np.array_equal(q, q_ref)
    deq = orc.dequant_rows(q, params, [0, x.shape[0]], bits, x.shape[1])
    assert np.all(np.abs(deq - RV[f"qrows{bits}_deq"]) <= dequant_atol(mn, sc, bits)[:, None])


def test_v1_vs_reference_x86_vectors():
    x, bits = RV["v1_x"], RV["v1_bits"]
    q, rng, params = orc.quant_v1(x, bits)
    assert np.array_equal(rng, RV["v1_range"])
    assert np.array_equal(params, RV["v1_params"])
    assert np.array_equal(q, RV["v1_q"])
    d = orc.dequant_v1(q, rng, params, x.shape[1])
    assert np.all(np.abs(d - RV["v1_deq"]) <= dequant_atol(params[:, 1], params[:, 2], params[:, 0])[:, None])


@pytest.mark.skipif(orc.ref_ops() is None, reason="oracle/_ref not built on this host")
@pytest.mark.parametrize("bits", [8, 4, 2])
def test_rows_vs_live_reference_extension(bits):
    ref = orc.ref_ops()
    g = torch.Generator().manual_seed(bits)
    n, F = 4333, 123  # the reference script's shape (tests/test_quantization_ops.py:9-10)
    x = torch.randn(n, F, generator=g)
    q, params = orc.quant_rows(x.numpy(), [0, n], bits)
    epb = 8 // bits
    q_ref = torch.zeros(((n + epb - 1) // epb) * F, dtype=torch.uint8)
    ref.quantize_tensor(x, q_ref, torch.from_numpy(params[:, 0].copy()), torch.from_numpy(params[:, 1].copy()), bits)
    assert np.array_equal(q.reshape(-1), q_ref.numpy())
    d_ref = torch.zeros(n, F)
    ref.dequantize_tensor(q_ref, d_ref, torch.from_numpy(params[:, 0].copy()), torch.from_numpy(params[:, 1].copy()), bits)
    d = orc.dequant_rows(q, params, [0, n], bits, F)
    assert np.all(np.abs(d - d_ref.numpy()) <= dequant_atol(params[:, 0], params[:, 1], bits)[:, None])
    # v1 with a uniform bit width: same params, same codes, feature-packed
    p3 = torch.zeros(n, 3); p3[:, 0] = bits
    rng = orc.v1_range([bits] * n, F)
    q1_ref = torch.zeros(int(rng[-1]), dtype=torch.uint8)
    ref.quantize_tensor_v1(x, q1_ref, torch.from_numpy(rng), p3)
    q1, rng1, p1 = orc.quant_v1(x.numpy(), [bits] * n)
    assert np.array_equal(q1, q1_ref.numpy()) and np.array_equal(p1, p3.numpy())


@pytest.mark.parametrize("bits", [8, 4, 2])
def test_codes_equal_torch_round_formula(bits):
    # independent one-liner: torch.round is round-half-to-even
    g = torch.Generator().manual_seed(100 + bits)
    x = torch.randn(257, 96, generator=g)
    x[::10] *= 100
    mn = x.min(dim=1, keepdim=True).values
    sc = (x.max(dim=1, keepdim=True).values - mn) / float(2 ** bits - 1)
    codes = torch.round((x - mn) / sc).to(torch.int64).numpy()
    q, params = orc.quant_rows(x.numpy(), [0, 257], bits)
    epb = 8 // bits
    for k in range(epb):
        rows = np.arange(k, 257, epb)
        got = (q[: len(rows)] >> ((epb - 1 - k) * bits)) & ((1 << bits) - 1)
        assert np.array_equal(got, codes[rows])
    assert np.array_equal(params[:, 0], mn.numpy()[:, 0]) and np.array_equal(params[:, 1], sc.numpy()[:, 0])


@pytest.mark.parametrize("bits", [8, 4, 2])
def test_segment_concatenation_invariant(bits):
    # tests/test_quantization_ops.py:214-228 of the reference:
    # for_all_procs(x, ranges) == cat_p quantize_tensor(x[range_p])
    rng = np.random.default_rng(bits)
    n, F, P = 1201, 40, 37
    x = rng.standard_normal((n, F), dtype=np.float32)
    cuts = np.sort(rng.integers(0, n, size=P - 1))
    seg = np.concatenate([[0], cuts, [n]]).astype(np.int32)  # includes empty segments now and then
    q, params = orc.quant_rows(x, seg, bits)
    parts, pparts = [], []
    for p in range(P):
        xs = np.ascontiguousarray(x[seg[p]:seg[p + 1]])
        qp, pp = orc.quant_rows(xs, [0, xs.shape[0]], bits)
        parts.append(qp); pparts.append(pp)
    assert np.array_equal(q, np.concatenate(parts, axis=0))
    assert np.array_equal(params, np.concatenate(pparts, axis=0))
    assert q.shape[0] == int(orc.packed_rows(seg, bits).sum())
    # numpy formulation agrees too
    q2, p2 = orc.quant_rows_numpy(x, seg, bits)
    assert np.array_equal(q, q2) and np.array_equal(params, p2)
    # round trip: |x_hat - x| <= scale/2 (+ rounding slack), row min recovered exactly
    d = orc.dequant_rows(q, params, seg, bits, F)
    assert np.all(np.abs(d - x) <= params[:, 1:2] * 0.5 * (1 + 1e-5) + 1e-6)
    assert np.array_equal(d.min(axis=1), x.min(axis=1))


def test_zero_sign_first_occurrence_and_constant_rows():
    # strict compares keep the FIRST of compare-equal values (quantization_arm.cpp:98-101)
    x = np.array([[0.0, -0.0, 1.0, 2.0], [-0.0, 0.0, 1.0, 2.0], [3.0, 3.0, 3.0, 3.0], [-0.0, -0.0, -0.0, -0.0],
                  [-1.0, -0.0, 0.0, -2.0]], dtype=np.float32)
    q, params = orc.quant_rows(x, [0, 5], 8)
    assert np.signbit(params[0, 0]) == False and np.signbit(params[1, 0]) == True  # noqa: E712
    assert params[2].tolist() == [3.0, 1.0] and q[2].tolist() == [0, 0, 0, 0]       # scale 0 -> 1
    assert np.signbit(params[3, 0]) and params[3, 1] == 1.0
    assert params[4, 0] == -2.0 and params[4, 1] == np.float32(2.0) / np.float32(255.0)


def test_denormal_and_large_scale():
    ulp = np.float32(2.0 ** -149)  # smallest fp32 denormal
    x = np.array([[0.0, 3 * ulp, 6 * ulp, 9 * ulp], [-3e38, 0.0, 1e38, 3e38]], dtype=np.float32)
    q, params = orc.quant_rows(x, [0, 2], 2)
    assert params[0, 1] == 3 * ulp  # a denormal scale, not flushed to zero (which would turn it into 1)
    codes0 = (q[0] >> 6) & 3
    assert codes0.tolist() == [0, 1, 2, 3]
