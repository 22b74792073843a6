"""Pins the CPU restatement of the SpMM path (oracle/sgnn_oracle.c) WITHOUT a GPU:
against the reference's own x86 extension when oracle/_ref is built, against scipy's CSR @ dense,
an fp64 accumulation, brute force, and algebraic invariants."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from oracle import oracle as orc
from _util import random_csr


def _ref_spmm(rowptr, col, val, x, out):
    ref = orc.ref_ops()
    T = torch.get_num_threads()
    M = rowptr.shape[0] - 1
    rs = torch.tensor(np.linspace(0, M, T + 1).astype(np.int32))
    cs = torch.tensor([0, x.shape[1]], dtype=torch.int32)
    o = torch.from_numpy(out)
    ref.spmm(torch.from_numpy(rowptr), torch.from_numpy(col), torch.from_numpy(val), torch.from_numpy(x), o, M, rs, cs)
    return out


needs_ref = pytest.mark.skipif(orc.ref_ops() is None, reason="oracle/_ref not built on this host")


@needs_ref
@pytest.mark.parametrize("M,K,F,deg", [(300, 200, 128, 9), (257, 100, 70, 5), (64, 64, 1, 3), (500, 400, 602, 4), (100, 50, 123, 20)])
def test_accumulate_bit_exact_vs_reference_extension(M, K, F, deg):
    rowptr, col, val = random_csr(M, K, deg, seed=M + F, empty_frac=0.2)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((K, F), dtype=np.float32)
    out0 = rng.standard_normal((M, F), dtype=np.float32)
    a = out0.copy(); orc.spmm_accumulate(rowptr, col, val, x, a)
    b = _ref_spmm(rowptr, col, val, x, out0.copy())
    assert np.array_equal(a, b)  # same fma sequence => same bits


@needs_ref
def test_overwrite_branch_vs_reference_extension():
    # sparsity <= 1e-4 and F > 256 selects the reference's generic overwrite kernel (spmm.cpp:601-602)
    M, K, F = 3000, 4000, 260
    rowptr, col, val = random_csr(M, K, 0.3, seed=5)
    assert orc.takes_overwrite_branch(int(rowptr[-1]), M, K, F)
    rng = np.random.default_rng(2)
    x = rng.standard_normal((K, F), dtype=np.float32)
    junk = rng.standard_normal((M, F), dtype=np.float32)
    a = junk.copy(); orc.spmm_dispatch(rowptr, col, val, x, a)
    b = _ref_spmm(rowptr, col, val, x, junk.copy())
    np.testing.assert_allclose(a, b, rtol=1e-6, atol=1e-7)  # contraction of acc + a*b is build dependent
    deg = np.diff(rowptr)
    assert np.all(a[deg == 0] == 0) and np.all(b[deg == 0] == 0)  # empty rows are zeroed, not skipped


@needs_ref
def test_dispatch_rule_vs_reference_extension():
    # just either side of both conditions: the reference result tells which branch it took
    for (M, K, F, deg) in [(2000, 3000, 257, 0.25), (2000, 3000, 256, 0.25), (200, 300, 300, 3.0)]:
        rowptr, col, val = random_csr(M, K, deg, seed=7)
        x = np.ones((K, F), dtype=np.float32)
        sentinel = np.full((M, F), 1000.0, dtype=np.float32)
        b = _ref_spmm(rowptr, col, val, x, sentinel.copy())
        ref_overwrote = bool(np.all(b[np.diff(rowptr) == 0] == 0)) and bool((np.diff(rowptr) == 0).any())
        assert orc.takes_overwrite_branch(int(rowptr[-1]), M, K, F) == ref_overwrote


def test_matches_scipy_and_fp64():
    M, K, F = 2000, 1500, 64
    rowptr, col, val = random_csr(M, K, 12, seed=11, empty_frac=0.1, hubs=3, hub_deg=900)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((K, F), dtype=np.float32)
    A = sp.csr_matrix((val, col, rowptr), shape=(M, K))
    want = A @ x
    got = np.zeros((M, F), dtype=np.float32); orc.spmm_accumulate(rowptr, col, val, x, got)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    got_o = np.full((M, F), 7.0, dtype=np.float32); orc.spmm_overwrite(rowptr, col, val, x, got_o)
    np.testing.assert_allclose(got_o, want, rtol=1e-5, atol=1e-5)
    f64 = orc.spmm_f64(rowptr, col, val, x)
    np.testing.assert_allclose(f64, A.astype(np.float64) @ x.astype(np.float64), rtol=1e-12, atol=1e-12)
    assert np.abs(got - f64).max() < 1e-3


def test_brute_force_tiny():
    rowptr = np.array([0, 2, 2, 5], dtype=np.int64)
    col = np.array([1, 0, 2, 2, 0], dtype=np.int64)  # row 2 has a duplicate edge to column 2
    val = np.array([0.5, 2.0, 1.0, 3.0, -1.0], dtype=np.float32)
    x = np.array([[1, 2], [3, 4], [5, 6]], dtype=np.float32)
    out = np.array([[10, 10], [20, 20], [30, 30]], dtype=np.float32)
    orc.spmm_accumulate(rowptr, col, val, x, out)
    want = np.array([[10 + 0.5 * 3 + 2 * 1, 10 + 0.5 * 4 + 2 * 2], [20, 20], [30 + 5 + 15 - 1, 30 + 6 + 18 - 2]], dtype=np.float32)
    assert np.array_equal(out, want)
    out2 = np.full((3, 2), 9.0, dtype=np.float32); orc.spmm_overwrite(rowptr, col, val, x, out2)
    assert np.array_equal(out2, want - np.array([[10], [20], [30]], dtype=np.float32))


def test_invariants_linearity_accumulate_transpose():
    M, K, F = 400, 300, 32
    rowptr, col, val = random_csr(M, K, 6, seed=21, empty_frac=0.3)
    rng = np.random.default_rng(4)
    x1 = rng.integers(-8, 8, (K, F)).astype(np.float32)  # small integers: every sum is exact in fp32
    x2 = rng.integers(-8, 8, (K, F)).astype(np.float32)
    vali = rng.integers(1, 4, val.shape).astype(np.float32)
    def run(x, init=None):
        o = np.zeros((M, F), np.float32) if init is None else init.copy()
        orc.spmm_accumulate(rowptr, col, vali, x, o); return o
    assert np.array_equal(run(x1 + x2), run(x1) + run(x2))
    init = rng.integers(-5, 5, (M, F)).astype(np.float32)
    assert np.array_equal(run(x1, init), init + run(x1))
    # empty rows untouched by the accumulate kernel
    empty = np.diff(rowptr) == 0
    assert empty.any() and np.array_equal(run(x1, init)[empty], init[empty])
    # backward == forward on the transpose (spmm_kernel.py:72-91)
    A = sp.csr_matrix((vali, col, rowptr), shape=(M, K))
    AT = A.T.tocsr(); AT.sort_indices()
    g = rng.integers(-8, 8, (M, F)).astype(np.float32)
    o = np.zeros((K, F), np.float32)
    orc.spmm_accumulate(AT.indptr.astype(np.int64), AT.indices.astype(np.int64), AT.data.astype(np.float32), g, o)
    assert np.array_equal(o, (A.T @ g).astype(np.float32))


def test_reference_test_recipe_shape():
    # tests/test_spmm.py:69-94 of the reference: 20020 x 1020, density 7e-4, F = 128, atol 1e-5
    A = sp.random(20020, 1020, density=0.0007, format="csr", dtype=np.float32, random_state=0)
    x = np.random.default_rng(0).random((1020, 128), dtype=np.float32)
    out = np.zeros((20020, 128), np.float32)
    orc.spmm_dispatch(A.indptr.astype(np.int64), A.indices.astype(np.int64), A.data, x, out)
    assert np.allclose(out, A @ x, atol=1e-5)


def test_row_divide_is_true_division():
    out = np.array([[1.0, 2.0], [3.0, 5.0]], dtype=np.float32)
    orc.row_divide(out, np.array([3.0, 7.0], dtype=np.float32))
    assert np.array_equal(out, np.array([[np.float32(1) / np.float32(3), np.float32(2) / np.float32(3)],
                                         [np.float32(3) / np.float32(7), np.float32(5) / np.float32(7)]], dtype=np.float32))


# ---- committed outputs of the reference's x86 extension (tests/golden/make_ref_vectors.py) ----------
import os  # noqa: E402

RV = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz"))


@pytest.mark.parametrize("tag", ["spmm_acc", "spmm_acc128"])
def test_accumulate_bit_exact_vs_committed_reference_vectors(tag):
    # runs on any host: no AVX-512 and no reference checkout needed
    rowptr, col, val, x = (RV[f"{tag}_{k}"] for k in ("rowptr", "col", "val", "x"))
    out = RV[f"{tag}_init"].copy()
    orc.spmm_accumulate(rowptr, col, val, x, out)
    assert np.array_equal(out, RV[f"{tag}_out"])
    assert not np.array_equal(out, RV[f"{tag}_init"])
    deg = np.diff(rowptr)
    assert np.array_equal(out[deg == 0], RV[f"{tag}_init"][deg == 0])


def test_overwrite_branch_vs_committed_reference_vectors():
    rowptr, col, val, x = (RV[f"spmm_ovw_{k}"] for k in ("rowptr", "col", "val", "x"))
    M, K, F = rowptr.shape[0] - 1, x.shape[0], x.shape[1]
    assert col.shape[0] >= 20 and orc.takes_overwrite_branch(col.shape[0], M, K, F)
    want = RV["spmm_ovw_out"]
    a = RV["spmm_ovw_init"].copy()
    orc.spmm_dispatch(rowptr, col, val, x, a)          # the dispatch rule must pick the overwrite kernel
    b = RV["spmm_ovw_init"].copy()
    orc.spmm_overwrite(rowptr, col, val, x, b)
    np.testing.assert_allclose(a, want, rtol=1e-6, atol=1e-7)
    assert np.array_equal(a, b)
    deg = np.diff(rowptr)
    assert np.all(want[deg == 0] == 0) and np.any(want[deg > 0] != 0)   # old contents discarded, empty rows zeroed
