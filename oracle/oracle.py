"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

ctypes front end of ``liborc.so`` (the plain-C CPU restatement in ``sgnn_oracle.c``) plus a
loader for the reference's own x86 extension when ``oracle/_ref`` has been built.  Only tests,
``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg import this module; nothing
under ``super_gnn_amd`` does.

All functions take contiguous numpy arrays and write their outputs in place, mirroring the
caller-allocates convention of the reference extension (super_gnn/ops/csrc/spmm.h:3-6,
super_gnn/ops/csrc/quantization_arm.h:5-10).
"""
import ctypes
import importlib.util
import os
import subprocess
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_i64p = ctypes.POINTER(ctypes.c_int64)
_i32p = ctypes.POINTER(ctypes.c_int32)
_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_u8p = ctypes.POINTER(ctypes.c_uint8)


def build(force=False):
    """Compile liborc.so with gcc (see Makefile)."""
    so = os.path.join(_HERE, "liborc.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.check_call(["make", "-C", _HERE, "liborc.so"], stdout=subprocess.DEVNULL)
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liborc.so")
        if not os.path.exists(so):
            build()
        L = ctypes.CDLL(so)
        L.orc_num_threads.restype = ctypes.c_int
        L.orc_set_num_threads.argtypes = [ctypes.c_int]
        L.orc_spmm_takes_overwrite_branch.restype = ctypes.c_int
        L.orc_spmm_takes_overwrite_branch.argtypes = [ctypes.c_int64] * 4
        for name in ("orc_spmm_accumulate", "orc_spmm_overwrite"):
            getattr(L, name).argtypes = [_i64p, _i64p, _f32p, _f32p, _f32p, ctypes.c_int64, ctypes.c_int64]
            getattr(L, name).restype = None
        L.orc_spmm_dispatch.argtypes = [_i64p, _i64p, _f32p, _f32p, _f32p] + [ctypes.c_int64] * 3
        L.orc_spmm_dispatch.restype = None
        L.orc_spmm_f64.argtypes = [_i64p, _i64p, _f32p, _f32p, _f32p, _f64p, ctypes.c_int64, ctypes.c_int64]
        L.orc_spmm_f64.restype = None
        L.orc_row_divide.argtypes = [_f32p, _f32p, ctypes.c_int64, ctypes.c_int64]
        L.orc_row_divide.restype = None
        L.orc_quant_rows.argtypes = [_f32p, _u8p, _f32p, _i32p, ctypes.c_int, ctypes.c_int64, ctypes.c_int]
        L.orc_quant_rows.restype = None
        L.orc_quant_rows_given_params.argtypes = [_f32p, _u8p, _f32p, _f32p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
        L.orc_quant_rows_given_params.restype = None
        L.orc_dequant_rows.argtypes = [_u8p, _f32p, _f32p, _i32p, ctypes.c_int, ctypes.c_int64, ctypes.c_int]
        L.orc_dequant_rows.restype = None
        L.orc_quant_v1.argtypes = [_f32p, _u8p, _i64p, _f32p, ctypes.c_int64, ctypes.c_int64]
        L.orc_quant_v1.restype = None
        L.orc_dequant_v1.argtypes = [_u8p, _f32p, _i64p, _f32p, ctypes.c_int64, ctypes.c_int64]
        L.orc_dequant_v1.restype = None
        _LIB = L
    return _LIB


def _p(a, dtype, ptype):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.dtype == dtype and a.flags.c_contiguous, (type(a), getattr(a, "dtype", None))
    return a.ctypes.data_as(ptype)


def num_threads():
    return lib().orc_num_threads()


def set_num_threads(n):
    lib().orc_set_num_threads(int(n))


def spmm_accumulate(rowptr, col, val, x, out):
    """out[m] += A[m,:] @ x for non-empty rows; see orc_spmm_accumulate."""
    M, F = out.shape
    lib().orc_spmm_accumulate(_p(rowptr, np.int64, _i64p), _p(col, np.int64, _i64p), _p(val, np.float32, _f32p),
                              _p(x, np.float32, _f32p), _p(out, np.float32, _f32p), M, F)


def spmm_overwrite(rowptr, col, val, x, out):
    M, F = out.shape
    lib().orc_spmm_overwrite(_p(rowptr, np.int64, _i64p), _p(col, np.int64, _i64p), _p(val, np.float32, _f32p),
                             _p(x, np.float32, _f32p), _p(out, np.float32, _f32p), M, F)


def spmm_dispatch(rowptr, col, val, x, out):
    M, F = out.shape
    lib().orc_spmm_dispatch(_p(rowptr, np.int64, _i64p), _p(col, np.int64, _i64p), _p(val, np.float32, _f32p),
                            _p(x, np.float32, _f32p), _p(out, np.float32, _f32p), M, x.shape[0], F)


def takes_overwrite_branch(nnz, M, K, F):
    return bool(lib().orc_spmm_takes_overwrite_branch(nnz, M, K, F))


def spmm_f64(rowptr, col, val, x, out_init=None):
    M, F = rowptr.shape[0] - 1, x.shape[1]
    out = np.empty((M, F), dtype=np.float64)
    lib().orc_spmm_f64(_p(rowptr, np.int64, _i64p), _p(col, np.int64, _i64p), _p(val, np.float32, _f32p),
                       _p(x, np.float32, _f32p), _p(out_init, np.float32, _f32p), _p(out, np.float64, _f64p), M, F)
    return out


def row_divide(out, deg):
    M, F = out.shape
    lib().orc_row_divide(_p(out, np.float32, _f32p), _p(deg, np.float32, _f32p), M, F)


def packed_rows(seg, bits):
    """Number of packed rows of each segment: ceil(n_p / (8/bits)) (super_gnn/quantizer.py:91-92)."""
    epb = 8 // bits
    seg = np.asarray(seg, dtype=np.int64)
    return (np.diff(seg) + epb - 1) // epb


def quant_rows(x, seg, bits):
    """Row-group quantize+pack. Returns (q u8[sum ceil(n_p/EPB), F], params f32[n, 2])."""
    n, F = x.shape
    seg = np.ascontiguousarray(seg, dtype=np.int32)
    P = seg.shape[0] - 1
    q = np.zeros((int(packed_rows(seg, bits).sum()), F), dtype=np.uint8)
    params = np.zeros((n, 2), dtype=np.float32)
    if n:
        lib().orc_quant_rows(_p(x, np.float32, _f32p), _p(q, np.uint8, _u8p), _p(params, np.float32, _f32p),
                             _p(seg, np.int32, _i32p), P, F, bits)
    return q, params


def quant_rows_given_params(x, mn, sc, bits):
    n, F = x.shape
    epb = 8 // bits
    q = np.zeros(((n + epb - 1) // epb, F), dtype=np.uint8)
    lib().orc_quant_rows_given_params(_p(x, np.float32, _f32p), _p(q, np.uint8, _u8p), _p(mn, np.float32, _f32p),
                                      _p(sc, np.float32, _f32p), n, F, bits)
    return q


def dequant_rows(q, params, seg, bits, F):
    seg = np.ascontiguousarray(seg, dtype=np.int32)
    P = seg.shape[0] - 1
    n = int(seg[-1])
    x = np.zeros((n, F), dtype=np.float32)
    if n:
        lib().orc_dequant_rows(_p(q, np.uint8, _u8p), _p(x, np.float32, _f32p), _p(params, np.float32, _f32p),
                               _p(seg, np.int32, _i32p), P, F, bits)
    return x


def v1_range(bits_per_row, F):
    """cumsum(ceil(b_i*F/8)) with a leading 0 (super_gnn/quantizer.py:66-73)."""
    b = np.asarray(bits_per_row, dtype=np.int64)
    r = np.zeros(b.shape[0] + 1, dtype=np.int64)
    np.cumsum((b * F + 7) // 8, out=r[1:])
    return r


def quant_v1(x, bits_per_row):
    n, F = x.shape
    rng = v1_range(bits_per_row, F)
    params = np.zeros((n, 3), dtype=np.float32)
    params[:, 0] = np.asarray(bits_per_row, dtype=np.float32)
    q = np.zeros(int(rng[-1]), dtype=np.uint8)
    lib().orc_quant_v1(_p(x, np.float32, _f32p), _p(q, np.uint8, _u8p), _p(rng, np.int64, _i64p),
                       _p(params, np.float32, _f32p), n, F)
    return q, rng, params


def dequant_v1(q, rng, params, F):
    n = params.shape[0]
    x = np.zeros((n, F), dtype=np.float32)
    lib().orc_dequant_v1(_p(q, np.uint8, _u8p), _p(x, np.float32, _f32p), _p(rng, np.int64, _i64p),
                         _p(params, np.float32, _f32p), n, F)
    return x


# ---------------------------------------------------------------------------------------------
# Independent numpy formulation of the row-group layout (vectorised, no shared code with the C
# file): used by tests to cross-check the C restatement, never by the product.
# ---------------------------------------------------------------------------------------------
def quant_rows_numpy(x, seg, bits):
    epb = 8 // bits
    qmax = np.float32((1 << bits) - 1)
    n, F = x.shape
    mn = x.min(axis=1) if n else np.zeros(0, np.float32)
    mx = x.max(axis=1) if n else np.zeros(0, np.float32)
    sc = ((mx - mn) / qmax).astype(np.float32)
    sc[sc == 0] = np.float32(1.0)
    codes = np.rint(((x - mn[:, None]).astype(np.float32) / sc[:, None]).astype(np.float32)).astype(np.uint32)
    outs = []
    for p in range(len(seg) - 1):
        c = codes[seg[p]:seg[p + 1]]
        pad = (-c.shape[0]) % epb
        c = np.concatenate([c, np.zeros((pad, F), np.uint32)], axis=0).reshape(-1, epb, F)
        shifts = ((epb - 1 - np.arange(epb)) * bits).astype(np.uint32)[None, :, None]
        outs.append(np.bitwise_or.reduce(c << shifts, axis=1).astype(np.uint8))
    q = np.concatenate(outs, axis=0) if outs else np.zeros((0, F), np.uint8)
    return q, np.stack([mn, sc], axis=1).astype(np.float32)


# ---------------------------------------------------------------------------------------------
# The reference's own x86 extension, when oracle/build_ref.sh has produced it.
# ---------------------------------------------------------------------------------------------
_REF = False


def ref_ops():
    """Return the reference extension module built into oracle/_ref, or None when it is absent
    or this host cannot run it (the build uses AVX-512 as the reference's setup.py does)."""
    global _REF
    if _REF is not False:
        return _REF
    _REF = None
    d = os.path.join(_HERE, "_ref")
    try:
        with open("/proc/cpuinfo") as f:
            if "avx512f" not in f.read():
                return None
    except OSError:
        return None
    if not os.path.isdir(d):
        return None
    cands = [f for f in os.listdir(d) if f.startswith("supergnn_ops") and f.endswith(".so")]
    if not cands:
        return None
    import torch  # noqa: F401  (the extension links libtorch)
    spec = importlib.util.spec_from_file_location("supergnn_ops", os.path.join(d, cands[0]))
    mod = importlib.util.module_from_spec(spec)
    try:
        spec.loader.exec_module(mod)
    except Exception as e:  # pragma: no cover
        print(f"oracle: reference extension present but not loadable: {e}", file=sys.stderr)
        return None
    _REF = mod
    return _REF
