"""MI355X-native implementation of SuperGNN's data-parallel hot path: CSR SpMM neighbour
aggregation and the boundary-row quantize / pack / unpack / dequantize pipeline, behind the
reference's own Python call signatures.  Importing this package loads libsgnn_hip.so and raises if
it is absent -- there is no CPU fallback."""
from . import _lib  # noqa: F401  (fails loudly when the HIP library is missing)
from . import supergnn_ops  # noqa: F401
from .ops.spmm_kernel import (SPMM_backward, SPMM_backward_quantized, SPMM_forward,  # noqa: F401
                              SPMM_forward_quantized)
from .quantizer import Quantizer_for_all_procs, QuantizerForMixedBits, QuantizerForPureBits  # noqa: F401
from .sparse import SparseTensor  # noqa: F401

__version__ = "0.1.0"
