"""``segment_csr(src, indptr, out, reduce)`` for reduce == 'sum' over a 1-D source: what
distribute_work_for_row asks of torch_scatter (super_gnn/ops/spmm_kernel.py:9)."""
import torch


def segment_csr(src, indptr, out=None, reduce="sum"):
    if reduce not in ("sum", "add"):
        raise NotImplementedError("only sum is provided")
    prefix = torch.zeros(src.shape[0] + 1, dtype=torch.float64, device=src.device)
    prefix[1:] = torch.cumsum(src.to(torch.float64), 0)
    res = (prefix[indptr[1:]] - prefix[indptr[:-1]]).to(src.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res
