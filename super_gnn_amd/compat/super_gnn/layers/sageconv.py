from super_gnn_amd.layers import DistSAGEConvGrad  # noqa: F401
