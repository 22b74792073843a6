from super_gnn_amd.aggregator import Aggregator  # noqa: F401
