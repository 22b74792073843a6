"""Minimal CSR matrix holder exposing the slice of the (forked) torch_sparse.SparseTensor interface
that the reference's SpMM façade touches (super_gnn/ops/spmm_kernel.py:46-91 and
tests/test_spmm.py:27-29): ``csr()``, ``coo()``, ``sparse_size(s)``, ``get/set_work_range``,
``get/set_work_range_for_transpose`` and ``storage.colptr()/row_T()/value_T()``.

It also owns what this build caches per matrix: the SpMM plans of A and of A^T."""
import numpy as np
import torch

from .supergnn_ops import SpmmPlan


class _Storage:
    def __init__(self, owner):
        self._o = owner

    def rowptr(self):
        return self._o._rowptr

    def col(self):
        return self._o._col

    def value(self):
        return self._o._value

    def colptr(self):
        self._o._build_transpose()
        return self._o._colptr

    def row_T(self):
        self._o._build_transpose()
        return self._o._row_T

    def value_T(self):
        self._o._build_transpose()
        return self._o._value_T


class SparseTensor:
    def __init__(self, row=None, rowptr=None, col=None, value=None, sparse_sizes=None, is_sorted=False):
        if col is None:
            raise ValueError("col is required")
        col = col.to(torch.int64)
        if sparse_sizes is None:
            raise ValueError("sparse_sizes is required")
        M, K = int(sparse_sizes[0]), int(sparse_sizes[1])
        if rowptr is None:
            if row is None:
                raise ValueError("row or rowptr is required")
            row = row.to(torch.int64)
            if not is_sorted:
                # stable sort by (row, col), as torch_sparse does on construction
                key = row * max(K, 1) + col
                perm = torch.argsort(key, stable=True)
                row, col = row[perm], col[perm]
                if value is not None:
                    value = value[perm]
            counts = torch.bincount(row, minlength=M)
            rowptr = torch.zeros(M + 1, dtype=torch.int64, device=col.device)
            torch.cumsum(counts, 0, out=rowptr[1:])
        self._rowptr = rowptr.to(torch.int64).contiguous()
        self._col = col.contiguous()
        self._value = value.contiguous() if value is not None else None
        self._sizes = (M, K)
        self._colptr = self._row_T = self._value_T = None
        self._work_range = (torch.empty(0, dtype=torch.int32), torch.empty(0, dtype=torch.int32))
        self._work_range_T = (torch.empty(0, dtype=torch.int32), torch.empty(0, dtype=torch.int32))
        self._plan = None
        self._plan_T = None
        self.storage = _Storage(self)

    # ---- construction helpers ---------------------------------------------------------------
    @classmethod
    def from_scipy(cls, mat):
        mat = mat.tocsr()
        mat.sort_indices()
        return cls(rowptr=torch.from_numpy(mat.indptr.astype(np.int64)),
                   col=torch.from_numpy(mat.indices.astype(np.int64)),
                   value=torch.from_numpy(np.ascontiguousarray(mat.data)), sparse_sizes=mat.shape, is_sorted=True)

    def to(self, device):
        out = SparseTensor(rowptr=self._rowptr.to(device), col=self._col.to(device),
                           value=self._value.to(device) if self._value is not None else None,
                           sparse_sizes=self._sizes, is_sorted=True)
        return out

    def cuda(self):
        return self.to(torch.device("cuda", torch.cuda.current_device()))

    def requires_grad_(self, flag=True):
        return self  # value gradients are not part of the aggregation path (spmm_value_bw_cpu is not exported)

    # ---- torch_sparse surface ---------------------------------------------------------------
    def csr(self):
        return self._rowptr, self._col, self._value

    def coo(self):
        counts = self._rowptr[1:] - self._rowptr[:-1]
        row = torch.repeat_interleave(torch.arange(self._sizes[0], device=self._col.device), counts)
        return row, self._col, self._value

    def sparse_size(self, dim):
        return self._sizes[dim]

    def sparse_sizes(self):
        return self._sizes

    def nnz(self):
        return self._col.numel()

    def to_dense(self):
        row, col, val = self.coo()
        out = torch.zeros(self._sizes, dtype=torch.float32 if val is None else val.dtype, device=col.device)
        out.index_put_((row, col), torch.ones_like(col, dtype=out.dtype) if val is None else val, accumulate=True)
        return out

    def get_work_range(self):
        return self._work_range

    def set_work_range(self, row_splits, col_splits):
        self._work_range = (row_splits, col_splits)

    def get_work_range_for_transpose(self):
        return self._work_range_T

    def set_work_range_for_transpose(self, row_splits, col_splits):
        self._work_range_T = (row_splits, col_splits)

    # ---- cached per-matrix state of this build ----------------------------------------------
    def _build_transpose(self):
        if self._colptr is not None:
            return
        row, col, val = self.coo()
        M, K = self._sizes
        perm = torch.argsort(col * max(M, 1) + row, stable=True)  # CSC order: by column, rows ascending
        self._row_T = row[perm].contiguous()
        self._value_T = val[perm].contiguous() if val is not None else None
        counts = torch.bincount(col, minlength=K)
        self._colptr = torch.zeros(K + 1, dtype=torch.int64, device=col.device)
        torch.cumsum(counts, 0, out=self._colptr[1:])

    def spmm_plan(self):
        if self._plan is None:
            self._plan = SpmmPlan(self._rowptr, self._col, self._sizes[1])
        return self._plan

    def spmm_plan_T(self):
        if self._plan_T is None:
            self._build_transpose()
            self._plan_T = SpmmPlan(self._colptr, self._row_T, self._sizes[0])
        return self._plan_T
