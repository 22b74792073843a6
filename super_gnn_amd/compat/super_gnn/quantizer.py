from super_gnn_amd.quantizer import Quantizer_for_all_procs, QuantizerForMixedBits, QuantizerForPureBits  # noqa: F401
