"""Shared helpers of the test-suite (inputs are seeded; nothing here touches the reference tree)."""
import numpy as np
import torch

from super_gnn_amd import synth


def random_csr(M, K, avg_deg, seed, empty_frac=0.0, hubs=0, hub_deg=0, dup=False):
    """Random CSR with optional empty rows, a few very long rows, and (optionally) duplicate edges.
    Returns numpy (rowptr int64, col int64, val float32)."""
    rng = np.random.default_rng(seed)
    deg = rng.poisson(avg_deg, size=M).astype(np.int64)
    if empty_frac > 0:
        deg[rng.random(M) < empty_frac] = 0
    if hubs:
        deg[rng.choice(M, size=min(hubs, M), replace=False)] = hub_deg
    rowptr = np.zeros(M + 1, dtype=np.int64)
    np.cumsum(deg, out=rowptr[1:])
    nnz = int(rowptr[-1])
    col = rng.integers(0, K, size=nnz, dtype=np.int64)
    if not dup:
        # sort inside each row (duplicates may remain; they are legal and must sum)
        row = np.repeat(np.arange(M), deg)
        order = np.lexsort((col, row))
        col = col[order]
    val = rng.random(nnz, dtype=np.float32)
    return rowptr, col, val


def to_np(t):
    return t.detach().cpu().numpy()


def graph_np(rowptr, col):
    return to_np(rowptr).astype(np.int64), to_np(col).astype(np.int64)


def gather_model_bytes(nnz, M, F, weighted=True, accumulate=True, mean=False):
    per_edge = 4 * F + 4 + (4 if weighted else 0)
    per_row = 4 * F + 8 + (4 * F if accumulate else 0) + (4 if mean else 0)
    return nnz * per_edge + M * per_row


def dequant_atol(zp, scale, bits):
    """Per-row absolute tolerance for dequantized floats.  code*scale + zp is computed with one
    rounding (fma) by some builds of the reference and two (mul, add) by others, so outputs may
    differ by one rounding of the larger intermediate: 2^-23 * (|zp| + qmax*|scale|)."""
    qmax = float((1 << int(bits)) - 1) if np.isscalar(bits) else (2.0 ** np.asarray(bits, dtype=np.float64) - 1)
    return (2.0 ** -23) * (np.abs(zp).astype(np.float64) + qmax * np.abs(scale).astype(np.float64)) + 1e-30


RTOL, ATOL = 1e-5, 1e-6  # the fp32 SpMM tolerance the task states


def abs_sum64(rowptr, col, val, x, init=None):
    """sum_e |val_e * x[col_e, f]| (+ |init|) in fp64: the scale of the rounding-error bound."""
    from oracle import oracle as orc
    v = np.abs(val) if val is not None else None
    return orc.spmm_f64(rowptr, col, v, np.abs(x), np.abs(init) if init is not None else None)


def assert_spmm_close(got, want, f64=None, abs_sum=None, deg=None, what=""):
    """Elementwise |gpu - ref32| <= 1e-6 + 1e-5*|ref32|.  Elements of LONG rows that miss it are
    adjudicated against the fp64 sum: two fp32 summation orders of n terms may legitimately differ
    by up to the forward error bound (n+1)*2^-24 * sum|terms| each (Higham, Accuracy and Stability
    of Numerical Algorithms, eq. 4.4), which for cancelling sums exceeds 1e-5 relative.  Such an
    element passes iff the GPU value meets that bound, and overall the GPU must not be less accurate
    than the sequential fp32 reference."""
    err = np.abs(got - want)
    tol = ATOL + RTOL * np.abs(want)
    bad = err > tol
    if bad.any() and f64 is not None:
        bound = (deg[:, None].astype(np.float64) + 1.0) * 2.0 ** -24 * abs_sum
        bad = bad & (np.abs(got - f64) > bound + ATOL)
        rms_gpu = np.sqrt(np.mean((got - f64) ** 2))
        rms_ref = np.sqrt(np.mean((want - f64) ** 2))
        assert rms_gpu <= 1.5 * rms_ref + 1e-7, f"{what}: gpu rms error {rms_gpu} vs reference fp32 {rms_ref}"
    assert not bad.any(), f"{what}: {bad.sum()} elements out of tolerance, max err {err.max()}"


