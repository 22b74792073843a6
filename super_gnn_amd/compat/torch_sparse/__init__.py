"""The slice of torch_sparse the SpMM façade and its test use."""
from super_gnn_amd.sparse import SparseTensor  # noqa: F401
from .matmul import matmul  # noqa: F401
