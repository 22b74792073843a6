"""Every diagnostic switch of the library (environment variables named SGNN_*; none is set in normal use) against
the CPU oracle: a switch only picks another kernel shape or schedule for the same arithmetic, so under each value
the SpMM must stay within the stated tolerance of the oracle (bit-identical where the schedule keeps the CSR edge
order), the quantizer's bytes and params must be the oracle's, and the fused product must equal dequantize-then-
multiply bit for bit.  All switches are read on every call (or, for the plan-shape ones, when the plan is built),
so one process can walk through them.  A second test checks that the sources name no switch this file does not
exercise."""
import glob
import os
import re

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from _util import random_csr, abs_sum64, assert_spmm_close

HERE = os.path.dirname(os.path.abspath(__file__))

# (variable, value, what it forces)
SPMM_SWITCHES = [
    ("SGNN_SPMM_BAND", "0", "never the band schedule"),
    ("SGNN_SPMM_BAND", "1", "band schedule for every fp32 product with column-sorted rows"),
    ("SGNN_SPMM_BAND_COLS", "96", "columns per band"),
    ("SGNN_SPMM_BAND_KB", "64", "per-XCD bytes of one band of the restaged operand"),
    ("SGNN_SPMM_BAND_SLICES", "2", "feature slices of a product that is not cut into windows"),
    ("SGNN_SPMM_BAND_SLICES", "1", "one feature slice"),
    ("SGNN_SPMM_BAND_CHUNK_ROWS", "3", "rows per chunk of the band kernel"),
    ("SGNN_SPMM_BAND_CHUNK_EDGES", "50", "staged edges per chunk (rounded down to a multiple of 16)"),
    ("SGNN_SPMM_BAND_OFF64", "1", "64-bit gather offsets in the band kernel"),
    ("SGNN_SPMM_BAND_WINDOW", "0", "wide products in one window"),
    ("SGNN_SPMM_BAND_WINDOW", "128", "windows of 128 feature columns"),
    ("SGNN_SPMM_HUB_LDS", "1", "long rows: one workgroup per row, partial sums reduced in LDS"),
    ("SGNN_SPMM_PARTITION", "0", "long rows not regrouped by column class"),
    ("SGNN_SPMM_PARTITION", "1", "long rows regrouped by column class"),
    ("SGNN_SPMM_PART_EDGES", "4000", "row blocks of at most this many edges"),
    ("SGNN_SPMM_SLICE", "0", "wide products in one piece"),
    ("SGNN_SPMM_SLICE", "64", "feature slices of 64 columns"),
]
QUANT_SWITCHES = [
    ("SGNN_QUANT_STREAM", "0", "lane-group quantizers at every width"),
    ("SGNN_QUANT_STREAM", "1", "stream quantizer at every width it can take"),
    ("SGNN_QUANT_EXACT_DIV", "1", "IEEE division for every element"),
    ("SGNN_DEQUANT_FLAT", "0", "row-tiled dequantizers"),
    ("SGNN_DEQUANT_ODD2", "0", "odd widths: four single floats per flat store"),
]


def _ops():
    import super_gnn_amd  # noqa: F401
    from super_gnn_amd import supergnn_ops
    return supergnn_ops


@pytest.mark.gpu
@pytest.mark.parametrize("name,value,what", SPMM_SWITCHES, ids=[f"{n}={v}" for n, v, _ in SPMM_SWITCHES])
def test_spmm_under_switch(name, value, what, monkeypatch):
    ops = _ops()
    dev = torch.device("cuda:0")
    if name.startswith("SGNN_SPMM_BAND_"):
        monkeypatch.setenv("SGNN_SPMM_BAND", "1")       # the band knobs shape a schedule that must first be taken
        if name != "SGNN_SPMM_BAND_COLS" and name != "SGNN_SPMM_BAND_KB":
            monkeypatch.setenv("SGNN_SPMM_BAND_COLS", "128")
    monkeypatch.setenv(name, value)
    M, K = 900, 1100
    rowptr, col, val = random_csr(M, K, 25, seed=len(name) + len(value), empty_frac=0.1, hubs=5, hub_deg=900)
    deg = np.diff(rowptr)
    for F in (128, 602, 37):
        rng = np.random.default_rng(F)
        x = rng.standard_normal((K, F), dtype=np.float32)
        init = rng.standard_normal((M, F), dtype=np.float32)
        plan = ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K)
        out = torch.from_numpy(init.copy()).to(dev)
        plan.run(torch.from_numpy(val).to(dev), torch.from_numpy(x).to(dev), out, accumulate=True)
        want = init.copy()
        orc.spmm_accumulate(rowptr, col, val, x, want)
        got = out.cpu().numpy()
        assert_spmm_close(got, want, orc.spmm_f64(rowptr, col, val, x, init), abs_sum64(rowptr, col, val, x, init), deg,
                          what=f"{name}={value} ({what}), F={F}")
        short = deg <= 128     # every schedule sums short rows in CSR order, one fma per edge
        assert np.array_equal(got[short], want[short]), f"{name}={value}, F={F}: short rows differ in bits"
        if plan.schedule(F)["band"] == 1:
            assert np.array_equal(got, want), f"{name}={value}, F={F}: the band schedule keeps CSR order on every row"
        # the fused product under the same switch: packed operand, same bits as dequantize-then-multiply
        if F % 2 == 0:
            seg = torch.tensor([0, K // 3, K], dtype=torch.int32)
            bits = 2 if F == 128 else 8
            epb = 8 // bits
            npk = sum(-(-(int(b) - int(a)) // epb) for a, b in zip(seg[:-1], seg[1:]))
            xd = torch.from_numpy(x).to(dev)
            q = torch.empty(npk, F, dtype=torch.uint8, device=dev)
            prm = torch.empty(K, 2, device=dev)
            ops.quantize_tensor_for_all_procs(xd, q, prm, seg, 2, bits)
            recv = torch.empty(K, F, device=dev)
            ops.dequantize_tensor_for_all_procs(q, recv, prm, seg, 2, bits)
            monkeypatch.setenv("SGNN_SPMM_BAND", "0")          # the separate product on the row-class kernels, like the fused one
            sep = torch.from_numpy(init.copy()).to(dev)
            ops.SpmmPlan(torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), K).run(
                torch.from_numpy(val).to(dev), recv, sep, accumulate=True)
            if name == "SGNN_SPMM_BAND" or name.startswith("SGNN_SPMM_BAND_"):
                monkeypatch.setenv("SGNN_SPMM_BAND", "1" if name != "SGNN_SPMM_BAND" else value)
            fused = torch.from_numpy(init.copy()).to(dev)
            plan.run_quantized(torch.from_numpy(val).to(dev), q, prm, ops.quant_segments(seg, bits), bits, fused, accumulate=True)
            if name in ("SGNN_SPMM_SLICE", "SGNN_SPMM_HUB_LDS"):   # (these two shape only the fp32 product: long rows sum in another order)
                rn = recv.cpu().numpy()
                assert_spmm_close(fused.cpu().numpy(), sep.cpu().numpy(), orc.spmm_f64(rowptr, col, val, rn, init),
                                  abs_sum64(rowptr, col, val, rn, init), deg, what=f"fused, {name}={value}, F={F}")
            else:
                assert torch.equal(fused, sep), f"{name}={value}, F={F}: fused differs from dequantize-then-multiply"


@pytest.mark.gpu
@pytest.mark.parametrize("name,value,what", QUANT_SWITCHES, ids=[f"{n}={v}" for n, v, _ in QUANT_SWITCHES])
def test_quantizer_under_switch(name, value, what, monkeypatch):
    ops = _ops()
    monkeypatch.setenv(name, value)
    n = 700
    seg = [0, 1, 9, 9, 300, n]
    seg_t = torch.tensor(seg, dtype=torch.int32)
    for F in (128, 100, 602, 123, 20, 1200):
        x = np.random.default_rng(F).standard_normal((n, F)).astype(np.float32)
        x[::7] *= 50.0
        x[5] = 2.0
        x[6, :3] = 0.0
        for bits in (8, 4, 2):
            q_ref, p_ref = orc.quant_rows(x, seg, bits)
            q = torch.full(q_ref.shape, 0xAB, dtype=torch.uint8, device="cuda")
            prm = torch.full((n, 2), -7.0, device="cuda")
            ops.quantize_tensor_for_all_procs(torch.from_numpy(x).cuda(), q, prm, seg_t, len(seg) - 1, bits)
            assert np.array_equal(prm.cpu().numpy().view(np.uint32), p_ref.view(np.uint32)), (name, value, F, bits)
            assert np.array_equal(q.cpu().numpy(), q_ref), (name, value, F, bits)
            d = torch.full((n, F), 123.0, device="cuda")
            ops.dequantize_tensor_for_all_procs(q, d, prm, seg_t, len(seg) - 1, bits)
            d_ref = orc.dequant_rows(q_ref, p_ref, np.asarray(seg, np.int64), bits, F)
            tol = (2.0 ** -23) * (np.abs(p_ref[:, :1]) + ((1 << bits) - 1) * np.abs(p_ref[:, 1:2])) + 1e-30
            assert np.all(np.abs(d.cpu().numpy().astype(np.float64) - d_ref) <= tol), (name, value, F, bits)


def test_every_switch_in_the_sources_is_exercised_here():
    named = set()
    for path in glob.glob(os.path.join(HERE, "..", "super_gnn_amd", "csrc", "*.h*")) + glob.glob(os.path.join(HERE, "..", "super_gnn_amd", "*.py")):
        named |= set(re.findall(r'"(SGNN_[A-Z0-9_]+)"', open(path).read()))
    covered = {n for n, _, _ in SPMM_SWITCHES + QUANT_SWITCHES}
    assert named <= covered, f"switches without a test: {sorted(named - covered)}"
    assert covered <= named, f"tests of switches that no longer exist: {sorted(covered - named)}"
    # no switch is latched at first use: a static initialised from getenv could not be walked through in one process
    for path in glob.glob(os.path.join(HERE, "..", "super_gnn_amd", "csrc", "*.h*")):
        assert not re.search(r"static\s+const[^;]*getenv", open(path).read()), path
