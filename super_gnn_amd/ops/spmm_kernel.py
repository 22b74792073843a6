"""SpMM façade with the reference's names and signatures (super_gnn/ops/spmm_kernel.py:46-91).

``SPMM_forward(src, other, out)``  : out += A @ other          (result in ``out``, returns None)
``SPMM_backward(src, other, out)`` : out += A^T @ other

The reference computes an nnz-balanced OpenMP row split on first use and caches it on the matrix
(spmm_kernel.py:49-58); here the object that matters is the GPU schedule (SpmmPlan), cached the same
way.  The row split is still computed once per matrix and stored through the work-range setters, so
callers that read ``get_work_range()`` see what the reference would have put there."""
import torch

from ..supergnn_ops import quant_segments, spmm


def distribute_work_for_row(rowptr: torch.Tensor, value: torch.Tensor, num_threads_on_row: int) -> torch.Tensor:
    """Greedy contiguous row split balanced by the per-row sum of ``value``: a range is closed at the
    first row whose addition lifts the running sum above total // threads, and that row opens the
    next range (super_gnn/ops/spmm_kernel.py:8-29).  The reference walks all rows in a Python loop;
    this finds each cut with one binary search over the prefix sums.  Kept for interface parity: the
    GPU kernels balance work through the SpMM plan instead and do not consume the split."""
    num_rows = rowptr.numel() - 1
    row_splits = torch.full((num_threads_on_row + 1,), num_rows, dtype=torch.int32)
    row_splits[0] = 0
    if num_rows == 0 or value is None or value.numel() == 0:
        return row_splits
    edge_prefix = torch.zeros(value.numel() + 1, dtype=torch.float64)
    edge_prefix[1:] = torch.cumsum(value.detach().to("cpu", torch.float64), 0)
    prefix = edge_prefix[rowptr.detach().cpu()]          # prefix[i] = sum of the first i rows
    target = float(torch.div(prefix[-1], num_threads_on_row, rounding_mode="floor"))
    start_sum, first_candidate = 0.0, 0                   # sum before the open range; earliest row that may close it
    for t in range(1, num_threads_on_row + 1):
        k = int(torch.searchsorted(prefix, torch.tensor(start_sum + target, dtype=torch.float64), right=True))
        cut = max(k - 1, first_candidate)                 # first row i with prefix[i+1] - start_sum > target
        if cut >= num_rows:
            break
        row_splits[t] = cut
        start_sum, first_candidate = float(prefix[cut]), cut + 1
    row_splits[-1] = num_rows
    return row_splits


def disribute_work_for_col(other: torch.Tensor, num_threads_on_col: int) -> torch.Tensor:
    """Even split of the feature axis (super_gnn/ops/spmm_kernel.py:31-44; the misspelt name is the
    reference's)."""
    num_cols = other.shape[-1]
    target = num_cols // num_threads_on_col
    col_splits = torch.full((num_threads_on_col + 1,), num_cols, dtype=torch.int32)
    for i in range(num_threads_on_col):
        col_splits[i] = i * target
    col_splits[-1] = num_cols
    return col_splits


def SPMM_forward(src, other: torch.Tensor, out: torch.Tensor, accumulate=None) -> None:
    """``accumulate=None`` follows the reference (out += A @ other except on its overwrite branch);
    ``False`` writes out = A @ other, which equals zero-filling out and accumulating, bit for bit,
    without the fill and the read-back."""
    rowptr, col, value = src.csr()
    col_splits = disribute_work_for_col(other, 1)
    row_splits, _ = src.get_work_range()
    if row_splits.size(0) == 0:   # once per matrix, as the reference does (spmm_kernel.py:49-53)
        row_splits = distribute_work_for_row(rowptr, value, torch.get_num_threads())
    src.set_work_range(row_splits, col_splits)
    if value is not None:
        value = value.to(other.dtype)
    sparse_row = rowptr.shape[0] - 1
    spmm(rowptr, col, value, other, out, sparse_row, row_splits, col_splits, plan=src.spmm_plan(), accumulate=accumulate)
    return None


def SPMM_backward(src, other: torch.Tensor, out: torch.Tensor, accumulate=None) -> None:
    colptr = src.storage.colptr()
    row_T = src.storage.row_T()
    value_T = src.storage.value_T()
    col_splits = disribute_work_for_col(other, 1)
    row_splits, _ = src.get_work_range_for_transpose()
    if row_splits.size(0) == 0:   # spmm_kernel.py:82-85
        row_splits = distribute_work_for_row(colptr, value_T, torch.get_num_threads())
    src.set_work_range_for_transpose(row_splits, col_splits)
    if value_T is not None:
        value_T = value_T.to(other.dtype)
    sparse_row = colptr.shape[0] - 1
    return spmm(colptr, row_T, value_T, other, out, sparse_row, row_splits, col_splits, plan=src.spmm_plan_T(),
                accumulate=accumulate)


def SPMM_forward_quantized(src, data_int8: torch.Tensor, quantized_params: torch.Tensor,
                           work_range_per_proc: torch.Tensor, num_bits: int, out: torch.Tensor) -> None:
    """out += A @ dequantize(data_int8), the remote / post-aggregation step of the forward pass with
    the boundary rows still packed: replaces ``Quantizer_for_all_procs.dequantize_intX_to_fp32(...)``
    followed by ``SPMM_forward(remote_adj_t, recv_buf, out)`` (super_gnn/aggregator.py:72-93) and
    gives the same floats, without materialising ``recv_buf``."""
    _, _, value = src.csr()
    if value is not None:
        value = value.to(torch.float32)
    segs = quant_segments(work_range_per_proc, num_bits)
    src.spmm_plan().run_quantized(value, data_int8, quantized_params, segs, num_bits, out, accumulate=True)
    return None


def SPMM_backward_quantized(src, data_int8: torch.Tensor, quantized_params: torch.Tensor,
                            work_range_per_proc: torch.Tensor, num_bits: int, out: torch.Tensor) -> None:
    """out += A^T @ dequantize(data_int8): the last step of the backward pass in pre/post-aggregation
    mode with the returned gradient rows still packed; replaces ``dequantize_intX_to_fp32(...)``
    followed by ``SPMM_backward(adj_t_pre_post_aggr_to, send_buf, local_grad)``
    (super_gnn/aggregator.py:159-171) and gives the same floats."""
    value_T = src.storage.value_T()
    if value_T is not None:
        value_T = value_T.to(torch.float32)
    segs = quant_segments(work_range_per_proc, num_bits)
    src.spmm_plan_T().run_quantized(value_T, data_int8, quantized_params, segs, num_bits, out, accumulate=True)
    return None
