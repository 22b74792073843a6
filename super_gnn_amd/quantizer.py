"""Quantizer façades with the reference's names and signatures (super_gnn/quantizer.py:10-92)."""
import math

import torch
from torch import Tensor

from . import supergnn_ops


class QuantizerForPureBits(object):
    """super_gnn/quantizer.py:10-47: one segment, row-group packed."""

    def __init__(self):
        pass

    @staticmethod
    def quantize_fp32_to_intX(data_fp32, data_intX, quant_params, num_bits=8):
        supergnn_ops.quantize_tensor(data_fp32, data_intX, quant_params, num_bits)

    @staticmethod
    def dequantize_intX_to_fp32(data_intX, data_fp32, dequant_params, num_bits=8):
        supergnn_ops.dequantize_tensor(data_intX, data_fp32, dequant_params, num_bits)

    @staticmethod
    def get_quantized_buffer_size(num_comm_nodes, num_bits, feat_len):
        return math.ceil(num_comm_nodes / float(8 / num_bits)) * feat_len


class QuantizerForMixedBits(object):
    """super_gnn/quantizer.py:50-73: per-row bit width, feature-packed."""

    @staticmethod
    def quantize_fp32_to_intX(data_fp32, data_int8, quantized_nodes_feat_range, quantized_params):
        supergnn_ops.quantize_tensor_v1(data_fp32, data_int8, quantized_nodes_feat_range, quantized_params)

    @staticmethod
    def dequantize_intX_to_fp32(data_int8, data_fp32, quantized_nodes_feat_range, dequantized_params):
        supergnn_ops.dequantize_tensor_v1(data_int8, data_fp32, quantized_nodes_feat_range, dequantized_params)

    @staticmethod
    def get_quantized_nodes_feat_range(num_nodes: int, feat_len: int, nodes_num_bits_tensor: Tensor):
        quantized_nodes_feat_len = torch.ceil(nodes_num_bits_tensor * feat_len / 8.0)
        quantized_nodes_feat_range = torch.empty((num_nodes + 1), dtype=torch.int64)
        quantized_nodes_feat_range[0] = 0
        torch.cumsum(quantized_nodes_feat_len, dim=0, out=quantized_nodes_feat_range[1:])
        return quantized_nodes_feat_range


class Quantizer_for_all_procs(object):
    """super_gnn/quantizer.py:75-92: the live training path; ``ctx`` is the process-wide instance
    other components look up (super_gnn/data_manager/CommSplits.py:15-16, super_gnn/aggregator.py:76)."""

    def __init__(self, world_size, num_bits) -> None:
        self.num_bits = num_bits
        self.world_size = world_size
        Quantizer_for_all_procs.ctx = self

    def quantize_fp32_to_intX(self, data_fp32, data_int8, quantized_params, quantized_work_range_per_proc):
        supergnn_ops.quantize_tensor_for_all_procs(data_fp32, data_int8, quantized_params,
                                                   quantized_work_range_per_proc, self.world_size, self.num_bits)

    def dequantize_intX_to_fp32(self, data_int8, data_fp32, quantized_params, dequantized_work_range_per_proc):
        supergnn_ops.dequantize_tensor_for_all_procs(data_int8, data_fp32, quantized_params,
                                                     dequantized_work_range_per_proc, self.world_size, self.num_bits)

    def get_quantized_splits(self, num_comm_nodes):
        return math.ceil(num_comm_nodes / float(8 / self.num_bits))
