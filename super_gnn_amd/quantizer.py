"""Quantizer façades: the three classes, method names and argument orders of the reference's
``super_gnn/quantizer.py`` (:10-47 pure bits, :50-73 mixed bits, :75-92 all-procs), running on the GPU
through ``super_gnn_amd.supergnn_ops``.  Buffers are caller-allocated and written in place."""
import torch
from torch import Tensor

from . import supergnn_ops as _ops


def _packed_rows(num_rows: int, num_bits: int) -> int:
    """ceil(num_rows / (8 / num_bits)): rows of the packed buffer that num_rows fp32 rows need."""
    rows_per_byte = 8 // int(num_bits)
    return -(-int(num_rows) // rows_per_byte)


class QuantizerForPureBits(object):
    """One segment, row-group packed (reference: super_gnn/quantizer.py:10-47)."""

    def __init__(self):
        pass

    @staticmethod
    def quantize_fp32_to_intX(data_fp32, data_intX, quant_params, num_bits=8):
        """data_intX u8[ceil(n/EPB)*F] and quant_params f32[n,2] = (zero_point, scale) are filled."""
        _ops.quantize_tensor(data_fp32, data_intX, quant_params, num_bits)

    @staticmethod
    def dequantize_intX_to_fp32(data_intX, data_fp32, dequant_params, num_bits=8):
        """data_fp32 f32[n,F] is filled from the packed codes and their per-row params."""
        _ops.dequantize_tensor(data_intX, data_fp32, dequant_params, num_bits)

    @staticmethod
    def get_quantized_buffer_size(num_comm_nodes, num_bits, feat_len):
        """Bytes of the packed buffer (super_gnn/quantizer.py:46-47)."""
        return _packed_rows(num_comm_nodes, num_bits) * feat_len


class QuantizerForMixedBits(object):
    """Per-row bit width, feature-packed (reference: super_gnn/quantizer.py:50-73)."""

    @staticmethod
    def quantize_fp32_to_intX(data_fp32, data_int8, quantized_nodes_feat_range, quantized_params):
        """quantized_params f32[n,3]: column 0 (bits) is read, columns 1-2 (zero_point, scale) written."""
        _ops.quantize_tensor_v1(data_fp32, data_int8, quantized_nodes_feat_range, quantized_params)

    @staticmethod
    def dequantize_intX_to_fp32(data_int8, data_fp32, quantized_nodes_feat_range, dequantized_params):
        _ops.dequantize_tensor_v1(data_int8, data_fp32, quantized_nodes_feat_range, dequantized_params)

    @staticmethod
    def get_quantized_nodes_feat_range(num_nodes: int, feat_len: int, nodes_num_bits_tensor: Tensor):
        """Byte range of every row in the ragged packed buffer: cumulative ceil(bits_i * feat_len / 8)
        with a leading 0, int64[num_nodes + 1] (super_gnn/quantizer.py:66-73)."""
        bits = nodes_num_bits_tensor.detach().to("cpu", torch.int64)
        row_bytes = torch.div(bits * int(feat_len) + 7, 8, rounding_mode="floor")
        out = torch.zeros(int(num_nodes) + 1, dtype=torch.int64)
        out[1:] = torch.cumsum(row_bytes[: int(num_nodes)], dim=0)
        return out


class Quantizer_for_all_procs(object):
    """The live training path (reference: super_gnn/quantizer.py:75-92): one packed segment per
    destination rank.  ``ctx`` is the process-wide instance other components look up
    (super_gnn/data_manager/CommSplits.py:15-16, super_gnn/aggregator.py:76)."""

    ctx = None

    def __init__(self, world_size, num_bits) -> None:
        self.world_size = world_size
        self.num_bits = num_bits
        type(self).ctx = self

    def quantize_fp32_to_intX(self, data_fp32, data_int8, quantized_params, quantized_work_range_per_proc,
                              row_index=None):
        """``quantized_params`` may be fp32 or bf16 pairs; with ``row_index`` the rows quantized are
        ``data_fp32[row_index]`` (see supergnn_ops.quantize_tensor_for_all_procs)."""
        _ops.quantize_tensor_for_all_procs(
            data_fp32, data_int8, quantized_params, quantized_work_range_per_proc, self.world_size, self.num_bits,
            row_index=row_index)

    def dequantize_intX_to_fp32(self, data_int8, data_fp32, quantized_params, dequantized_work_range_per_proc):
        _ops.dequantize_tensor_for_all_procs(
            data_int8, data_fp32, quantized_params, dequantized_work_range_per_proc, self.world_size, self.num_bits)

    def get_quantized_splits(self, num_comm_nodes):
        """Packed rows a segment of num_comm_nodes rows occupies (super_gnn/quantizer.py:91-92)."""
        return _packed_rows(num_comm_nodes, self.num_bits)
