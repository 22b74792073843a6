"""``super_gnn`` name shim: only the hot-path modules exist (ops.spmm_kernel, quantizer)."""
