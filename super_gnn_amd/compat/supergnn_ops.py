"""``import supergnn_ops`` -> the GPU implementation (same callables as the reference's native module,
super_gnn/ops/csrc/ops.cpp:13-28)."""
from super_gnn_amd.supergnn_ops import *  # noqa: F401,F403
from super_gnn_amd.supergnn_ops import (dequantize_tensor, dequantize_tensor_for_all_procs,  # noqa: F401
                                        dequantize_tensor_v1, quantize_tensor, quantize_tensor_for_all_procs,
                                        quantize_tensor_v1, spmm)
