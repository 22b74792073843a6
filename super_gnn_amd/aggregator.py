"""The aggregation data flow of the reference's ``Aggregator`` (super_gnn/aggregator.py:15-177) for P
vertex partitions that all live in ONE process on ONE GPU, with a loop-back exchange in place of the
all-to-all of super_gnn/communicator.py:221-306.

Per partition and direction the steps and their order are the reference's:

  forward  (aggregator.py:33-93)          pre-aggregation SpMM (or row gather) into send_buf
                                           -> quantize+pack per destination segment
                                           -> exchange -> local SpMM
                                           -> remote rows accumulated onto the same out
  backward (aggregator.py:98-177)          transposed SpMM of the remote graph into recv_buf
                                           -> quantize+pack -> exchange (reverse direction)
                                           -> local transposed SpMM -> accumulate the returned rows

Because the partitions share one process, the exchange is a set of device copies between their
buffers, and the phases run for all partitions before the next phase starts.  With num_bits in
{8,4,2} the receiver never materialises the fp32 rows: it feeds the packed bytes straight into the
fused unpack+dequantize+SpMM kernel (forward), which is bit-identical to dequantizing first.
"""
from typing import List, Sequence

import torch

from .ops.spmm_kernel import SPMM_backward, SPMM_forward, SPMM_forward_quantized
from .quantizer import Quantizer_for_all_procs


def _cumulative(splits):
    out = [0]
    for n in splits:
        out.append(out[-1] + n)
    return out


def _exchange(graphs, direction: str, quantized: bool, params_wire_dtype=None):
    """Loop-back all-to-all.  forward: rank p's send segment for r -> rank r's recv segment from p.
    backward: rank r's recv-side segment for p travels back into rank p's send-side segment for r
    (the reference reuses the same buffers with the roles swapped, aggregator.py:113-118,153-166)."""
    P = len(graphs)
    for p in range(P):
        gp = graphs[p]
        s_off = _cumulative(gp.comm_splits.send_splits)
        s_off_q = _cumulative(gp.comm_splits.send_splits_int2) if quantized else None
        for r in range(P):
            n = gp.comm_splits.send_splits[r]
            if n == 0 or p == r:
                continue
            gr = graphs[r]
            r_off = _cumulative(gr.comm_splits.recv_splits)
            assert gr.comm_splits.recv_splits[p] == n
            if not quantized:
                a = gp.comm_buf.send_buf[s_off[r]:s_off[r + 1]]
                b = gr.comm_buf.recv_buf[r_off[p]:r_off[p + 1]]
                (b.copy_(a) if direction == "forward" else a.copy_(b))
                continue
            r_off_q = _cumulative(gr.comm_splits.recv_splits_int2)
            qp, qr = gp.comm_buf_for_quantization, gr.comm_buf_for_quantization
            da = qp.quantized_send_data_buf[s_off_q[r]:s_off_q[r + 1]]
            db = qr.quantized_recv_data_buf[r_off_q[p]:r_off_q[p + 1]]
            pa = qp.quantized_send_params_buf_fp32[s_off[r]:s_off[r + 1]]
            pb = qr.quantized_recv_params_buf_fp32[r_off[p]:r_off[p + 1]]
            src_d, dst_d, src_p, dst_p = (da, db, pa, pb) if direction == "forward" else (db, da, pb, pa)
            dst_d.copy_(src_d)
            if params_wire_dtype is not None:  # the reference ships params as bf16 (communicator.py:283-294)
                dst_p.copy_(src_p.to(params_wire_dtype).to(torch.float32))
            else:
                dst_p.copy_(src_p)


class LoopbackAggregator(torch.autograd.Function):
    """``outs = LoopbackAggregator.apply(world, *feats)`` with ``world = LoopbackWorld(...)``;
    ``feats[p]`` are partition p's node features [n_p, F] on the GPU, ``outs[p]`` its aggregated rows."""

    @staticmethod
    def forward(ctx, world, *feats):
        graphs, bits, pre = world.graphs, world.num_bits, world.is_pre_delay
        quantized = bits in (2, 4, 8)
        F = feats[0].shape[-1]
        qz = Quantizer_for_all_procs(len(graphs), bits) if quantized else None
        for g, x in zip(graphs, feats):
            g.comm_buf.resize_buffer(g.comm_splits, F, bits)
            if quantized:
                g.comm_buf_for_quantization.resize_buffer(g.comm_splits, F, bits)
            send_buf = g.comm_buf.send_buf
            send_buf.zero_()                                              # aggregator.py:41
            if send_buf.shape[0]:
                if pre:
                    SPMM_forward(g.adj_t_pre_post_aggr_to, x, send_buf)   # aggregator.py:46
                else:
                    torch.index_select(x, 0, g.idx_nodes_send_to_others, out=send_buf)   # aggregator.py:48
                if quantized:                                             # communicator.py:269
                    q = g.comm_buf_for_quantization
                    qz.quantize_fp32_to_intX(send_buf, q.quantized_send_data_buf, q.quantized_send_params_buf_fp32,
                                             q.quantized_work_range_per_proc)
        _exchange(graphs, "forward", quantized, world.params_wire_dtype)
        outs = []
        for g, x in zip(graphs, feats):
            out = torch.zeros((g.local_adj_t.sparse_size(0), F), dtype=torch.float32, device=x.device)
            SPMM_forward(g.local_adj_t, x, out)                           # aggregator.py:62-65
            remote = g.adj_t_pre_post_aggr_from if pre else g.remote_adj_t
            if remote.sparse_size(1):
                if quantized and F % 4 == 0:
                    q = g.comm_buf_for_quantization                       # fused: aggregator.py:72-93 in one pass
                    SPMM_forward_quantized(remote, q.quantized_recv_data_buf, q.quantized_recv_params_buf_fp32,
                                           q.dequantized_work_range_per_proc, bits, out)
                else:
                    if quantized:
                        q = g.comm_buf_for_quantization
                        qz.dequantize_intX_to_fp32(q.quantized_recv_data_buf, g.comm_buf.recv_buf,
                                                   q.quantized_recv_params_buf_fp32, q.dequantized_work_range_per_proc)
                    SPMM_forward(remote, g.comm_buf.recv_buf, out)         # aggregator.py:90/92
            outs.append(out)
        ctx.world = world
        return tuple(outs)

    @staticmethod
    def backward(ctx, *grads):
        world = ctx.world
        graphs, bits, pre = world.graphs, world.num_bits, world.is_pre_delay
        quantized = bits in (2, 4, 8)
        F = grads[0].shape[-1]
        qz = Quantizer_for_all_procs(len(graphs), bits) if quantized else None
        for g, go in zip(graphs, grads):
            go = go.contiguous()
            g.comm_buf.resize_buffer(g.comm_splits, F, bits)
            if quantized:
                g.comm_buf_for_quantization.resize_buffer(g.comm_splits, F, bits)
            recv_buf = g.comm_buf.recv_buf
            recv_buf.zero_()                                              # aggregator.py:122
            if recv_buf.shape[0]:
                remote = g.adj_t_pre_post_aggr_from if pre else g.remote_adj_t
                SPMM_backward(remote, go, recv_buf)                       # aggregator.py:125/127
                if quantized:                                             # the reverse trip is quantized too
                    q = g.comm_buf_for_quantization
                    qz.quantize_fp32_to_intX(recv_buf, q.quantized_recv_data_buf, q.quantized_recv_params_buf_fp32,
                                             q.dequantized_work_range_per_proc)
        _exchange(graphs, "backward", quantized, world.params_wire_dtype)
        outs = []
        for g, go in zip(graphs, grads):
            go = go.contiguous()
            local_grad = torch.zeros((g.local_adj_t.sparse_size(1), F), dtype=torch.float32, device=go.device)
            SPMM_backward(g.local_adj_t, go, local_grad)                  # aggregator.py:145-148
            send_buf = g.comm_buf.send_buf
            if send_buf.shape[0]:
                if quantized:                                             # aggregator.py:159-164
                    q = g.comm_buf_for_quantization
                    qz.dequantize_intX_to_fp32(q.quantized_send_data_buf, send_buf, q.quantized_send_params_buf_fp32,
                                               q.quantized_work_range_per_proc)
                if pre:
                    SPMM_backward(g.adj_t_pre_post_aggr_to, send_buf, local_grad)          # aggregator.py:171
                else:
                    local_grad.index_add_(0, g.idx_nodes_send_to_others, send_buf)           # aggregator.py:173-175
            outs.append(local_grad)
        return (None,) + tuple(outs)


class LoopbackWorld(object):
    """The P partitions of one graph plus the aggregation settings the reference passes per call
    (num_bits, is_pre_delay).  ``params_wire_dtype=torch.bfloat16`` reproduces the reference's bf16
    transport of (zero_point, scale) (communicator.py:283-294); None keeps them fp32."""

    def __init__(self, graphs: Sequence[object], num_bits: int, is_pre_delay: bool, params_wire_dtype=None) -> None:
        self.graphs = list(graphs)
        self.num_bits = int(num_bits)
        self.is_pre_delay = bool(is_pre_delay)
        self.params_wire_dtype = params_wire_dtype

    def aggregate(self, feats: Sequence[torch.Tensor]) -> List[torch.Tensor]:
        return list(LoopbackAggregator.apply(self, *feats))
