"""Drop-in for the reference's native module ``supergnn_ops`` (super_gnn/ops/csrc/ops.cpp:13-28),
running on one MI355X through libsgnn_hip.so.

Same callables, same argument order, same in-place / returns-None convention as the build the
reference's Python code calls (the ARM arities, super_gnn/ops/csrc/quantization_arm.h:5-10 and
super_gnn/ops/csrc/spmm.h:3-6):

    spmm(rowptr, col, value, mat, out, sparse_rows, row_split, col_split)
    quantize_tensor(input, output, quantized_params, bits)
    dequantize_tensor(input, output, quantized_params, bits)
    quantize_tensor_for_all_procs(input, output, quantized_params, work_range_per_proc, num_procs, bits)
    dequantize_tensor_for_all_procs(input, output, dequantized_params, work_range_per_proc, num_procs, bits)
    quantize_tensor_v1(input, output, quantized_nodes_feat_range, quantized_params)
    dequantize_tensor_v1(input, output, quantized_nodes_feat_range, quantized_params)

Deliberate differences from the reference, all on the side of failing loudly:
  * wrong dtypes raise TypeError (the reference prints and returns without computing, spmm.cpp:530-535);
  * column indices and row pointers are range-checked once per matrix;
  * quantize_tensor / dequantize_tensor honour ``bits`` (the ARM build hard-codes 2,
    quantization_arm.cpp:447-448; the x86 build honours it, quantization_x86.cpp:33).

Tensors on the GPU are used in place (zero copy, on the current stream).  CPU tensors -- what the
reference's own tests create -- are staged to the GPU, and the result is copied back into the
caller's output storage.  Nothing is ever computed on the CPU.
"""
import ctypes
from collections import OrderedDict

import torch

from . import _lib
from ._lib import check, lib

__all__ = [
    "spmm", "quantize_tensor", "dequantize_tensor", "quantize_tensor_for_all_procs",
    "dequantize_tensor_for_all_procs", "quantize_tensor_v1", "dequantize_tensor_v1",
    "SpmmPlan", "quant_segments", "spmm_dequantized",
]


def _device():
    if not torch.cuda.is_available():
        raise RuntimeError("super_gnn_amd needs a GPU (MI355X / gfx950); there is no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current stream's hipStream_t (the raw getter is ~8 us cheaper per call than the Stream object)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _want(t, dtype, name):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")


class _Staged:
    """Device view of a caller tensor.  A GPU tensor is used as is; a CPU tensor is copied to the
    GPU and, for outputs, copied back into the caller's storage on commit()."""

    def __init__(self, t, dev, writeback=False):
        self.orig = t
        self.writeback = False
        if t.is_cuda:
            if not t.is_contiguous():
                if writeback:
                    raise ValueError("output tensors on the GPU must be contiguous")
                t = t.contiguous()
            self.dev = t.detach()
        else:
            self.dev = t.detach().contiguous().to(dev)
            self.writeback = writeback

    def commit(self):
        if self.writeback:
            with torch.no_grad():
                self.orig.copy_(self.dev)


# -------------------------------------------------------------------------------------------------
# SpMM
# -------------------------------------------------------------------------------------------------
class SpmmPlan:
    """Per-matrix schedule (see sgnn_spmm_plan in include/sgnn.h).  Holds device copies of rowptr
    and 32-bit column indices plus the long-row segments; build once, reuse every call -- the role
    row_splits play in the reference (super_gnn/ops/spmm_kernel.py:49-58)."""

    def __init__(self, rowptr, col, num_cols, long_row_threshold=0, piece_edges=0):
        _want(rowptr, torch.int64, "rowptr")
        if col.dtype not in (torch.int64, torch.int32):
            raise TypeError(f"col must be int64 or int32, got {col.dtype}")
        dev = _device()
        rp = rowptr.contiguous().to(dev)
        cl = col.contiguous().to(dev)
        self.M = rp.numel() - 1
        self.K = int(num_cols)
        self.nnz = cl.numel()
        if self.M < 0:
            raise ValueError("rowptr must have at least one entry")
        _destroy_plan_handle()   # handles parked during a graph capture
        h = ctypes.c_void_p()
        check(lib.sgnn_spmm_plan_create(_ptr(rp), _ptr(cl), int(cl.dtype == torch.int64), self.M, self.K, self.nnz,
                                        int(long_row_threshold), int(piece_edges), _stream(), ctypes.byref(h)))
        self._h = h
        self._bound = None   # (value tensor, version) whose long-row values the plan holds in its own order
        self._seen = None    # (value tensor, version) of the previous call
        self._bound_slots = None  # row-slot table (a tensor owned by a _Segments object) bound to the plan
        self.device = dev

    def info(self):
        buf = (ctypes.c_int64 * 10)()
        check(lib.sgnn_spmm_plan_info(self._h, buf))
        keys = ("M", "K", "nnz", "long_rows", "pieces", "long_edges", "long_row_threshold", "piece_edges",
                "partitioned", "top_share_ppm")
        return dict(zip(keys, list(buf)))

    def schedule(self, F):
        """Which schedule a product of feature width F takes (sgnn_spmm_plan_schedule)."""
        buf = (ctypes.c_int64 * 4)()
        check(lib.sgnn_spmm_plan_schedule(self._h, int(F), buf))
        return dict(zip(("band", "band_cols", "n_bands", "n_slices"), list(buf)))

    def run(self, value, mat, out, accumulate=True, row_div=None):
        """out (+)= A @ mat on the current stream.  value None = all ones."""
        _want(mat, torch.float32, "mat")
        _want(out, torch.float32, "out")
        if value is not None:
            _want(value, torch.float32, "value")
            if value.numel() != self.nnz:
                raise ValueError(f"value has {value.numel()} entries, the matrix has {self.nnz}")
        if mat.dim() != 2 or out.dim() != 2:
            raise ValueError("mat and out must be 2-D")
        if mat.shape[0] != self.K:
            raise ValueError(f"mat has {mat.shape[0]} rows, the sparse matrix has {self.K} columns")
        if out.shape[0] != self.M or out.shape[1] != mat.shape[1]:
            raise ValueError(f"out must be [{self.M}, {mat.shape[1]}], got {list(out.shape)}")
        if row_div is not None:
            _want(row_div, torch.float32, "row_div")
            if row_div.numel() != self.M:
                raise ValueError("row_div must have one entry per sparse row")
        dev = self.device
        s_val = _Staged(value, dev) if value is not None else None
        s_mat = _Staged(mat, dev)
        s_out = _Staged(out, dev, writeback=True)
        s_div = _Staged(row_div, dev) if row_div is not None else None
        F = mat.shape[1]
        if value is not None and value.is_cuda and value.is_contiguous():
            self._maybe_bind(value)
        check(lib.sgnn_spmm_csr_f32(self._h, _ptr(s_val.dev) if s_val else None, _ptr(s_mat.dev), _ptr(s_out.dev),
                                    F, F, F, int(bool(accumulate)), _ptr(s_div.dev) if s_div else None, _stream()))
        s_out.commit()

    def _maybe_bind(self, value):
        """Edge values that come back unchanged are bound to the plan on their second use: the plan
        then keeps the long rows' values in its own edge order (sgnn_spmm_plan_bind_values).

        "Unchanged" = same address and same version counter as a tensor this plan still holds a
        reference to (so the address cannot have been recycled; a view of it shares its counter).
        Anything else at the bound address is rebound at once, so the library never reads a stale
        copy."""
        def same(ref):
            return ref is not None and value.data_ptr() == ref[0].data_ptr() and value._version == ref[1]
        if same(self._bound):
            return
        stale = self._bound is not None and value.data_ptr() == self._bound[0].data_ptr()
        if stale or same(self._seen):
            check(lib.sgnn_spmm_plan_bind_values(self._h, _ptr(value), _stream()))
            self._bound = (value, value._version)
        self._seen = (value, value._version)

    def bind_values(self, value):
        """Bind (or re-bind) an edge-value tensor by hand.  run() does this by itself for a tensor that comes
        back unchanged, and notices edits that move the tensor's version counter; call this after changing the
        values in a way the counter does not see (a write through ``.data``, a kernel given the raw pointer)."""
        _want(value, torch.float32, "value")
        if not (value.is_cuda and value.is_contiguous() and value.numel() == self.nnz):
            raise ValueError("value must be a contiguous GPU tensor with one entry per edge")
        check(lib.sgnn_spmm_plan_bind_values(self._h, _ptr(value), _stream()))
        self._bound = self._seen = (value, value._version)

    def unbind_values(self):
        """Forget the bound edge values: every later product reads the tensor it is given."""
        check(lib.sgnn_spmm_plan_bind_values(self._h, None, _stream()))
        self._bound = self._seen = None

    def run_quantized(self, value, data_int8, params, segs, bits, out, accumulate=True, row_div=None):
        """out (+)= A @ dequantize(data_int8): the dense operand stays packed (row-group layout,
        ``segs`` from quant_segments()) and is decoded inside the gather."""
        _check_bits(bits)
        _want(data_int8, torch.uint8, "data_int8")
        bf16 = _params_kind(params, "quantized_params")
        _want(out, torch.float32, "out")
        if value is not None:
            _want(value, torch.float32, "value")
            if value.numel() != self.nnz:
                raise ValueError(f"value has {value.numel()} entries, the matrix has {self.nnz}")
        if out.dim() != 2 or out.shape[0] != self.M:
            raise ValueError(f"out must be [{self.M}, F]")
        F = out.shape[1]
        if F % 2:
            raise ValueError("the fused path needs an even feature width")
        if segs.n_rows != self.K:
            raise ValueError(f"the segment table covers {segs.n_rows} rows, the sparse matrix has {self.K} columns")
        if data_int8.numel() < segs.n_packed * F or params.numel() < self.K * 2:
            raise ValueError("packed data / params smaller than the segment table requires")
        if not (data_int8.is_cuda and params.is_cuda and out.is_cuda and (value is None or value.is_cuda)):
            raise ValueError("the fused path takes GPU tensors only")
        if not (data_int8.is_contiguous() and params.is_contiguous() and out.is_contiguous()):
            raise ValueError("tensors must be contiguous")
        if row_div is not None:
            _want(row_div, torch.float32, "row_div")
        slots = segs.row_slots(bits)
        if slots is not None and self._bound_slots is not slots:
            # the segment table of a partition never changes: carry each edge's slot with its column
            check(lib.sgnn_spmm_plan_bind_row_slots(self._h, _ptr(slots), _stream()))
            self._bound_slots = slots
        if value is not None and value.is_contiguous():
            self._maybe_bind(value)
        if bf16:
            check(lib.sgnn_spmm_csr_dq_wire_f32(self._h, _ptr(value), _ptr(data_int8), _ptr(params), 1, _ptr(slots), bits,
                                                _ptr(out), F, F, int(bool(accumulate)), _ptr(row_div), _stream()))
        else:
            check(lib.sgnn_spmm_csr_dq_f32(self._h, _ptr(value), _ptr(data_int8), _ptr(params), _ptr(slots), bits,
                                           _ptr(out), F, F, int(bool(accumulate)), _ptr(row_div), _stream()))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        destroy = _destroy_plan_handle    # None once the interpreter has begun to tear the module down
        if h and destroy is not None:
            destroy(h)


# Plan handles whose owner died while a stream was being captured into a HIP graph.  Destroying a plan frees
# device memory, and a free issued during a capture invalidates the capture (Python's cyclic collector may run a
# plan's finaliser at any allocation, i.e. also in the middle of somebody's ``torch.cuda.graph`` block), so such
# handles wait here until the next plan is created or destroyed outside a capture.
_deferred_handles = []


def _capturing():
    try:
        return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()
    except Exception:
        return False


def _destroy_plan_handle(h=None):
    try:
        if _capturing():
            if h:
                _deferred_handles.append(h)
            return
        if h:
            lib.sgnn_spmm_plan_destroy(h)
        while _deferred_handles:
            lib.sgnn_spmm_plan_destroy(_deferred_handles.pop())
    except Exception:
        pass


def _cached_plan(rowptr, col, K):
    """Plan cached ON the rowptr tensor object (the reference caches its row split on the matrix
    object the same way).  The entry pins the col tensor it was built from and both version
    counters, so a recycled allocation or an in-place edit can never alias a stale plan."""
    entries = rowptr.__dict__.setdefault("_sgnn_plans", [])
    for e in entries:
        if e[0] is col and e[1] == (rowptr._version, col._version, int(K)):
            return e[2]
    plan = SpmmPlan(rowptr, col, K)
    entries[:] = [e for e in entries if e[0] is not col][-3:]
    entries.append((col, (rowptr._version, col._version, int(K)), plan))
    return plan


def reference_overwrites(nnz, M, K, F):
    """True when the reference's spmm() takes its overwrite branch (spmm.cpp:601-602)."""
    return bool(lib.sgnn_spmm_reference_overwrites(int(nnz), int(M), int(K), int(F)))


def spmm(rowptr, col, value, mat, out, sparse_rows, row_split=None, col_split=None, *, plan=None, accumulate=None,
         row_div=None):
    """supergnn_ops.spmm (super_gnn/ops/csrc/spmm.cpp:594-608): result in ``out``, returns None.

    Accumulates into ``out`` unless the reference's dispatch rule selects its overwrite branch
    (nnz/M/K <= 1e-4 and F > 256); ``accumulate=True/False`` forces a mode.  ``row_split`` /
    ``col_split`` (the reference's OpenMP work ranges) are accepted and ignored.  ``plan`` lets
    callers that own the matrix pass its cached SpmmPlan; otherwise one is cached per
    (rowptr, col) storage."""
    if value is None:
        # spmm.cpp:398 dereferences the optional unconditionally on the branch it would take.
        raise TypeError("value is required (use ones for an unweighted graph)")
    if rowptr.numel() - 1 != int(sparse_rows):
        raise ValueError(f"sparse_rows={sparse_rows} but rowptr has {rowptr.numel()} entries")
    K = mat.shape[0]
    if plan is None:
        plan = _cached_plan(rowptr, col, K)
    if accumulate is None:
        accumulate = not reference_overwrites(col.numel(), sparse_rows, K, mat.shape[1])
    plan.run(value, mat, out, accumulate=accumulate, row_div=row_div)
    return None


# -------------------------------------------------------------------------------------------------
# Row-group quantization
# -------------------------------------------------------------------------------------------------
class _Segments:
    def __init__(self, seg_host, bits, dev):
        P = seg_host.numel() - 1
        seg_host = seg_host.to(torch.int32).contiguous()
        pseg_host = torch.empty(P + 1, dtype=torch.int32)
        total = lib.sgnn_quant_segment_offsets(
            ctypes.cast(seg_host.data_ptr(), ctypes.POINTER(ctypes.c_int32)), P, bits,
            ctypes.cast(pseg_host.data_ptr(), ctypes.POINTER(ctypes.c_int32)))
        check(total)
        self.P = P
        self.n_rows = int(seg_host[-1])
        self.n_packed = int(total)
        self.seg = seg_host.to(dev)
        self.pseg = pseg_host.to(dev)
        self.pseg_host = pseg_host
        self.seg_host = seg_host
        self._slots = None

    def row_slots(self, bits):
        """Device table row -> position in the padded row space, or None when it is the identity
        (every segment but the last holds a multiple of EPB rows)."""
        epb = 8 // bits
        sizes = (self.seg_host[1:] - self.seg_host[:-1])[:-1]
        if self.P == 1 or bool((sizes % epb == 0).all()):
            return None
        if self._slots is None:
            self._slots = torch.empty(self.n_rows, dtype=torch.int32, device=self.seg.device)
            check(lib.sgnn_quant_row_slots(_ptr(self.seg), _ptr(self.pseg), self.P, bits, self.n_rows,
                                           _ptr(self._slots), _stream()))
        return self._slots


def quant_segments(work_range, bits):
    """Device copies of the segment table and its packed-row offsets, cached on the tensor object
    (keyed by its version counter, so in-place edits rebuild them)."""
    _want(work_range, torch.int32, "work_range_per_proc")
    dev = _device()
    cache = work_range.__dict__.setdefault("_sgnn_segments", {})
    key = (int(bits), work_range._version, str(dev))
    s = cache.get(key)
    if s is None:
        cache.clear()
        s = _Segments(work_range.detach().cpu(), int(bits), dev)
        cache[key] = s
    return s


def _check_bits(bits):
    if bits not in (2, 4, 8):
        raise ValueError(f"bits={bits}: only 8, 4 and 2 pack into bytes")  # TORCH_CHECK(8 % bits == 0), quantization_arm.cpp:438


def _params_kind(params, name):
    """0 for fp32 (zero_point, scale) pairs, 1 for the bf16 pairs the reference puts on the wire
    (super_gnn/communicator.py:283-294)."""
    if params.dtype == torch.float32:
        return 0
    if params.dtype == torch.bfloat16:
        return 1
    raise TypeError(f"{name} must be torch.float32 or torch.bfloat16, got {params.dtype}")


def _checked_row_index(row_index, n_src):
    """An int64 GPU index tensor whose range has been checked once (cached on the tensor object)."""
    _want(row_index, torch.int64, "row_index")
    if row_index.dim() != 1 or not row_index.is_contiguous():
        raise ValueError("row_index must be a contiguous 1-D tensor")
    seen = row_index.__dict__.get("_sgnn_index_ok")
    if seen != (row_index._version, int(n_src)):
        if row_index.numel() and (int(row_index.min()) < 0 or int(row_index.max()) >= n_src):
            raise IndexError(f"row_index out of range for a source of {n_src} rows")
        row_index.__dict__["_sgnn_index_ok"] = (row_index._version, int(n_src))
    return row_index


def _quant_rows(inp, out_u8, params, segs, bits, row_index=None):
    _want(inp, torch.float32, "input")
    _want(out_u8, torch.uint8, "output")
    bf16 = _params_kind(params, "quantized_params")
    if inp.dim() != 2:
        raise ValueError("input must be [rows, features]")
    if row_index is not None:
        return _quant_gathered_rows(inp, row_index, out_u8, params, bf16, segs, bits)
    n, F = inp.shape
    if segs.n_rows != n:
        raise ValueError(f"segment table ends at row {segs.n_rows}, input has {n} rows")
    if out_u8.numel() < segs.n_packed * F:
        raise ValueError(f"output holds {out_u8.numel()} bytes, {segs.n_packed * F} needed")
    if params.numel() < n * 2:
        raise ValueError(f"quantized_params holds {params.numel()} floats, {n * 2} needed")
    dev = _device()
    s_in = _Staged(inp, dev)
    s_q = _Staged(out_u8, dev, writeback=True)
    s_p = _Staged(params, dev, writeback=True)
    if bf16:
        check(lib.sgnn_quant_pack_rows_wire_f32(_ptr(s_in.dev), F, None, n, _ptr(s_q.dev), _ptr(s_p.dev), 1, _ptr(segs.seg),
                                                _ptr(segs.pseg), segs.P, n, segs.n_packed, F, bits, _stream()))
    else:
        check(lib.sgnn_quant_pack_rows_f32(_ptr(s_in.dev), _ptr(s_q.dev), _ptr(s_p.dev), _ptr(segs.seg), _ptr(segs.pseg),
                                           segs.P, n, segs.n_packed, F, bits, _stream()))
    s_q.commit()
    s_p.commit()


def _quant_gathered_rows(src, row_index, out_u8, params, bf16, segs, bits):
    """Quantize rows src[row_index[r]] without materialising them (GPU tensors only)."""
    if not (src.is_cuda and row_index.is_cuda and out_u8.is_cuda and params.is_cuda):
        raise ValueError("the gathering quantizer takes GPU tensors only")
    if src.stride(1) != 1 or not (out_u8.is_contiguous() and params.is_contiguous()):
        raise ValueError("input rows must be dense (unit stride) and outputs contiguous")
    n_src, F = src.shape
    n = row_index.numel()
    _checked_row_index(row_index, n_src)
    if segs.n_rows != n:
        raise ValueError(f"segment table ends at row {segs.n_rows}, row_index has {n} entries")
    if out_u8.numel() < segs.n_packed * F:
        raise ValueError(f"output holds {out_u8.numel()} bytes, {segs.n_packed * F} needed")
    if params.numel() < n * 2:
        raise ValueError(f"quantized_params holds {params.numel()} elements, {n * 2} needed")
    check(lib.sgnn_quant_pack_rows_wire_f32(_ptr(src), src.stride(0), _ptr(row_index), n_src, _ptr(out_u8), _ptr(params),
                                            bf16, _ptr(segs.seg), _ptr(segs.pseg), segs.P, n, segs.n_packed, F, bits,
                                            _stream()))


def _dequant_rows(inp_u8, out, params, segs, bits):
    _want(inp_u8, torch.uint8, "input")
    _want(out, torch.float32, "output")
    bf16 = _params_kind(params, "dequantized_params")
    if out.dim() != 2:
        raise ValueError("output must be [rows, features]")
    n, F = out.shape
    if segs.n_rows != n:
        raise ValueError(f"segment table ends at row {segs.n_rows}, output has {n} rows")
    if inp_u8.numel() < segs.n_packed * F:
        raise ValueError(f"input holds {inp_u8.numel()} bytes, {segs.n_packed * F} needed")
    if params.numel() < n * 2:
        raise ValueError(f"dequantized_params holds {params.numel()} floats, {n * 2} needed")
    dev = _device()
    s_q = _Staged(inp_u8, dev)
    s_p = _Staged(params, dev)
    s_out = _Staged(out, dev, writeback=True)
    if bf16:
        check(lib.sgnn_unpack_dequant_rows_wire_f32(_ptr(s_q.dev), _ptr(s_out.dev), _ptr(s_p.dev), 1, _ptr(segs.seg),
                                                    _ptr(segs.pseg), segs.P, n, segs.n_packed, F, bits, _stream()))
    else:
        check(lib.sgnn_unpack_dequant_rows_f32(_ptr(s_q.dev), _ptr(s_out.dev), _ptr(s_p.dev), _ptr(segs.seg),
                                               _ptr(segs.pseg), segs.P, n, segs.n_packed, F, bits, _stream()))
    s_out.commit()


_SINGLE_SEG = OrderedDict()


def _single_segment(n, bits):
    key = (int(n), int(bits), str(_device()))
    s = _SINGLE_SEG.get(key)
    if s is None:
        s = _Segments(torch.tensor([0, int(n)], dtype=torch.int32), int(bits), _device())
        _SINGLE_SEG[key] = s
        while len(_SINGLE_SEG) > 64:
            _SINGLE_SEG.popitem(last=False)
    return s


def quantize_tensor(input, output, quantized_params, bits):
    """quantize_tensor (quantization_arm.cpp:433-464): one segment; output u8[ceil(n/EPB)*F]."""
    _check_bits(bits)
    _quant_rows(input, output, quantized_params, _single_segment(input.shape[0], bits), bits)


def dequantize_tensor(input, output, quantized_params, bits):
    """dequantize_tensor (quantization_arm.cpp:466-494)."""
    _check_bits(bits)
    _dequant_rows(input, output, quantized_params, _single_segment(output.shape[0], bits), bits)


def quantize_tensor_for_all_procs(input, output, quantized_params, work_range_per_proc, num_procs, bits,
                                  row_index=None):
    """quantize_tensor_for_all_procs (quantization_arm.cpp:496-578): segment p = rows
    [work_range[p], work_range[p+1]) is packed on its own, starting at packed row
    sum_{q<p} ceil(n_q / EPB).

    Beyond the reference's arguments: ``quantized_params`` may be a bfloat16 tensor (the (zero_point,
    scale) pairs are then stored in the wire format of super_gnn/communicator.py:283-294, codes still
    computed from the fp32 values), and ``row_index`` (int64, GPU) makes row r of the quantizer's
    input ``input[row_index[r]]`` -- the index_select into send_buf of super_gnn/aggregator.py:48
    folded into the quantizer."""
    _check_bits(bits)
    if work_range_per_proc.numel() != int(num_procs) + 1:
        raise ValueError("work_range_per_proc must have num_procs + 1 entries")
    _quant_rows(input, output, quantized_params, quant_segments(work_range_per_proc, bits), bits, row_index=row_index)


def dequantize_tensor_for_all_procs(input, output, dequantized_params, work_range_per_proc, num_procs, bits):
    """dequantize_tensor_for_all_procs (quantization_arm.cpp:580-633)."""
    _check_bits(bits)
    if work_range_per_proc.numel() != int(num_procs) + 1:
        raise ValueError("work_range_per_proc must have num_procs + 1 entries")
    _dequant_rows(input, output, dequantized_params, quant_segments(work_range_per_proc, bits), bits)


def spmm_dequantized(rowptr, col, value, data_int8, quantized_params, work_range_per_proc, num_procs, bits, out,
                     *, plan=None, accumulate=True, row_div=None):
    """out (+)= A @ dequantize(data_int8) in one pass (no reference counterpart as a single call:
    it fuses dequantize_tensor_for_all_procs with the spmm that follows it in
    super_gnn/aggregator.py:72-93).  A has one column per quantized row."""
    if work_range_per_proc.numel() != int(num_procs) + 1:
        raise ValueError("work_range_per_proc must have num_procs + 1 entries")
    segs = quant_segments(work_range_per_proc, bits)
    if plan is None:
        plan = _cached_plan(rowptr, col, segs.n_rows)
    plan.run_quantized(value, data_int8, quantized_params, segs, bits, out, accumulate=accumulate, row_div=row_div)
    return None


# -------------------------------------------------------------------------------------------------
# Feature-packed mixed-bit quantization
# -------------------------------------------------------------------------------------------------
def _v1_common(fp32, u8, rng, params, fp32_name):
    _want(fp32, torch.float32, fp32_name)
    _want(u8, torch.uint8, "packed data")
    _want(rng, torch.int64, "quantized_nodes_feat_range")
    _want(params, torch.float32, "quantized_params")
    if fp32.dim() != 2:
        raise ValueError(f"{fp32_name} must be [rows, features]")
    n, F = fp32.shape
    if rng.numel() != n + 1:
        raise ValueError("quantized_nodes_feat_range must have rows + 1 entries")
    if params.numel() != n * 3:
        raise ValueError("quantized_params must be [rows, 3] = (bits, zero_point, scale)")
    # The layout check below reads the GPU (it is what keeps a bad range from writing out of bounds); it
    # is done once per (range, params) pair and version, cached on the range tensor object.
    seen = rng.__dict__.get("_sgnn_v1_checked")
    key = (rng._version, params._version, int(u8.numel()), int(F))
    if seen is not None and seen[0] is params and seen[1] == key:
        return n, F
    if n:
        bits = params.detach().reshape(n, 3)[:, 0]
        ok = (bits == 8) | (bits == 4) | (bits == 2)
        if not bool(ok.all()):
            raise ValueError("per-row bits must be 8, 4 or 2")
        need = torch.div(bits.to(torch.int64) * F + 7, 8, rounding_mode="floor")
        r = rng.detach().to(bits.device)
        if not bool(((r[1:] - r[:-1]) >= need).all()) or int(r[-1]) > u8.numel() or int(r[0]) < 0:
            raise ValueError("quantized_nodes_feat_range does not fit the per-row bit widths / packed buffer")
    rng.__dict__["_sgnn_v1_checked"] = (params, key)
    return n, F


def quantize_tensor_v1(input, output, quantized_nodes_feat_range, quantized_params):
    """quantize_tensor_v1 (quantization_arm.cpp:635-702): per-row bit width read from
    quantized_params[:, 0]; zero_point / scale written to columns 1 and 2."""
    n, F = _v1_common(input, output, quantized_nodes_feat_range, quantized_params, "input")
    dev = _device()
    s_in = _Staged(input, dev)
    s_q = _Staged(output, dev, writeback=True)
    s_r = _Staged(quantized_nodes_feat_range, dev)
    s_p = _Staged(quantized_params, dev, writeback=True)
    check(lib.sgnn_quant_v1_f32(_ptr(s_in.dev), _ptr(s_q.dev), _ptr(s_r.dev), _ptr(s_p.dev), n, F, _stream()))
    s_q.commit()
    s_p.commit()


def dequantize_tensor_v1(input, output, quantized_nodes_feat_range, quantized_params):
    """dequantize_tensor_v1 (quantization_arm.cpp:704-757)."""
    n, F = _v1_common(output, input, quantized_nodes_feat_range, quantized_params, "output")
    dev = _device()
    s_q = _Staged(input, dev)
    s_r = _Staged(quantized_nodes_feat_range, dev)
    s_p = _Staged(quantized_params, dev)
    s_out = _Staged(output, dev, writeback=True)
    check(lib.sgnn_dequant_v1_f32(_ptr(s_q.dev), _ptr(s_out.dev), _ptr(s_r.dev), _ptr(s_p.dev), n, F, _stream()))
    s_out.commit()
