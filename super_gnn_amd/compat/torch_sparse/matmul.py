"""``matmul(src, other, reduce)``: CSR x dense on the GPU with autograd for the dense operand
(the gradient is the transposed product, as SPMM_backward computes it)."""
import torch

from super_gnn_amd.ops.spmm_kernel import SPMM_backward, SPMM_forward


class _SpMM(torch.autograd.Function):
    @staticmethod
    def forward(ctx, src, other):
        ctx.src = src
        out = torch.zeros((src.sparse_size(0), other.shape[-1]), dtype=other.dtype, device=other.device)
        SPMM_forward(src, other.detach(), out)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        src = ctx.src
        grad = torch.zeros((src.sparse_size(1), grad_out.shape[-1]), dtype=grad_out.dtype, device=grad_out.device)
        SPMM_backward(src, grad_out.contiguous(), grad)
        return None, grad


def matmul(src, other, reduce="sum"):
    if reduce not in ("sum", "add"):
        raise NotImplementedError("only sum aggregation is on the hot path (mean = sum / degree in the layer)")
    return _SpMM.apply(src, other)
