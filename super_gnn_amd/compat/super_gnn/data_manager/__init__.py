from super_gnn_amd.data_manager import (CommBuffer, CommBufferForQuantization, CommSplits, DistributedGraph,  # noqa: F401
                                        DistributedGraphForPre)
