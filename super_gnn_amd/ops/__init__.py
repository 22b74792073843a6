from .spmm_kernel import SPMM_forward, SPMM_backward, SPMM_forward_quantized  # noqa: F401
