from super_gnn_amd.sparse import SparseTensor  # noqa: F401
