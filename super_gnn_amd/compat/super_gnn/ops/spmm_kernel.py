from super_gnn_amd.ops.spmm_kernel import (SPMM_backward, SPMM_forward, SPMM_forward_quantized,  # noqa: F401
                                           disribute_work_for_col, distribute_work_for_row)
