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

What is folded together on the GPU (each fold gives the floats of the unfolded sequence):

  * with num_bits in {8,4,2} the receiver never materialises fp32 rows: the packed bytes go straight
    into the fused unpack+dequantize+SpMM kernel, forward (remote graph) and backward (transposed
    pre-aggregation graph, or the 0/1 selection matrix that stands for ``index_add_``);
  * in the plain mode the boundary rows are quantized straight out of the feature matrix
    (``index_select`` folded into the quantizer's loads);
  * (zero_point, scale) can be produced and consumed as bf16 pairs, the reference's wire format;
  * "zero the buffer, then accumulate A @ x into it" is one overwriting SpMM (same floats: the sum
    starts from 0 either way; rows without edges are written as zeros).

Because the partitions share one process, every partition's buffers are slices of one arena per
buffer kind, and the exchange is ONE row-permuting copy per buffer (send rows of all ranks -> recv
rows of all ranks).  The send-side chain and the local SpMMs are issued on two streams.
"""
from typing import List, Sequence

import torch

from .ops.spmm_kernel import (SPMM_backward, SPMM_backward_quantized, SPMM_forward, SPMM_forward_quantized)
from .quantizer import Quantizer_for_all_procs
from .sparse import SparseTensor


def _cumulative(splits):
    out = [0]
    for n in splits:
        out.append(out[-1] + n)
    return out


class _Arena(object):
    """Buffers of all partitions for one feature width, and the row permutations of the exchange."""

    def __init__(self, graphs, F, quantized, params_dtype, device, half=False):
        self.F, self.quantized, self.params_dtype, self.half = F, quantized, params_dtype, half
        self.send_tot = _cumulative([sum(g.comm_splits.send_splits) for g in graphs])
        self.recv_tot = _cumulative([sum(g.comm_splits.recv_splits) for g in graphs])
        n = self.send_tot[-1]
        assert n == self.recv_tot[-1]
        self.send = torch.zeros((n, F), dtype=torch.float32, device=device)
        self.recv = torch.zeros((n, F), dtype=torch.float32, device=device)
        self.perm = self._permutation(graphs, "send_splits", "recv_splits", self.send_tot, self.recv_tot, device)
        self.inv_perm = torch.empty_like(self.perm)
        self.inv_perm[self.perm] = torch.arange(n, device=device)
        if half:  # the 16-bit mode ships bf16 copies of the rows (CommBuffer.py:11-17, communicator.py:101-127)
            self.send16 = torch.zeros((n, F), dtype=torch.bfloat16, device=device)
            self.recv16 = torch.zeros((n, F), dtype=torch.bfloat16, device=device)
        if not quantized:
            return
        self.qs_tot = _cumulative([sum(g.comm_splits.send_splits_int2) for g in graphs])
        self.qr_tot = _cumulative([sum(g.comm_splits.recv_splits_int2) for g in graphs])
        nq = self.qs_tot[-1]
        self.send_q = torch.zeros((nq, F), dtype=torch.uint8, device=device)
        self.recv_q = torch.zeros((nq, F), dtype=torch.uint8, device=device)
        self.send_params = torch.zeros((n, 2), dtype=params_dtype, device=device)
        self.recv_params = torch.zeros((n, 2), dtype=params_dtype, device=device)
        self.perm_q = self._permutation(graphs, "send_splits_int2", "recv_splits_int2", self.qs_tot, self.qr_tot, device)
        self.inv_perm_q = torch.empty_like(self.perm_q)
        self.inv_perm_q[self.perm_q] = torch.arange(nq, device=device)
        # one (zero_point, scale) pair moves as one machine word
        word = torch.int64 if params_dtype == torch.float32 else torch.int32
        self.send_params_w = self.send_params.view(word)
        self.recv_params_w = self.recv_params.view(word)

    def bind(self, graphs):
        """Point every partition's buffer attributes at its slices of this arena."""
        for p, g in enumerate(graphs):
            s0, s1, r0, r1 = self.send_tot[p], self.send_tot[p + 1], self.recv_tot[p], self.recv_tot[p + 1]
            g.comm_buf.send_buf, g.comm_buf.recv_buf = self.send[s0:s1], self.recv[r0:r1]
            if self.half:
                g.comm_buf.send_buf_fp16, g.comm_buf.recv_buf_fp16 = self.send16[s0:s1], self.recv16[r0:r1]
            if not self.quantized:
                continue
            q = g.comm_buf_for_quantization
            q.quantized_send_data_buf = self.send_q[self.qs_tot[p]:self.qs_tot[p + 1]]
            q.quantized_recv_data_buf = self.recv_q[self.qr_tot[p]:self.qr_tot[p + 1]]
            q.send_params, q.recv_params = self.send_params[s0:s1], self.recv_params[r0:r1]
            if self.params_dtype == torch.float32:
                q.quantized_send_params_buf_fp32, q.quantized_recv_params_buf_fp32 = q.send_params, q.recv_params
            else:
                q.quantized_send_params_buf_bf16, q.quantized_recv_params_buf_bf16 = q.send_params, q.recv_params

    @staticmethod
    def _permutation(graphs, send_name, recv_name, send_tot, recv_tot, device):
        """perm[j] = row of the send arena that lands in row j of the recv arena (all_to_all_single
        semantics: rank p's segment for r becomes rank r's segment from p)."""
        P = len(graphs)
        perm = torch.empty(recv_tot[-1], dtype=torch.int64)
        send_cum = [_cumulative(getattr(g.comm_splits, send_name)) for g in graphs]
        for r, g in enumerate(graphs):
            recv_cum = _cumulative(getattr(g.comm_splits, recv_name))
            for p in range(P):
                n = recv_cum[p + 1] - recv_cum[p]
                assert n == send_cum[p][r + 1] - send_cum[p][r]
                if n:
                    begin = send_tot[p] + send_cum[p][r]
                    perm[recv_tot[r] + recv_cum[p]:recv_tot[r] + recv_cum[p + 1]] = torch.arange(begin, begin + n)
        return perm.to(device)

    def exchange(self, direction, quantized):
        if direction == "forward":
            if quantized:
                torch.index_select(self.send_q, 0, self.perm_q, out=self.recv_q)
                torch.index_select(self.send_params_w, 0, self.perm, out=self.recv_params_w)
            elif self.half:  # send_buf_fp16.copy_(send_buf); all_to_all; recv_buf.copy_(recv_buf_fp16)
                self.send16.copy_(self.send)
                torch.index_select(self.send16, 0, self.perm, out=self.recv16)
                self.recv.copy_(self.recv16)
            else:
                torch.index_select(self.send, 0, self.perm, out=self.recv)
        else:  # the same buffers with the roles swapped (aggregator.py:113-118,153-166)
            if quantized:
                torch.index_select(self.recv_q, 0, self.inv_perm_q, out=self.send_q)
                torch.index_select(self.recv_params_w, 0, self.inv_perm, out=self.send_params_w)
            elif self.half:
                self.recv16.copy_(self.recv)
                torch.index_select(self.recv16, 0, self.inv_perm, out=self.send16)
                self.send.copy_(self.send16)
            else:
                torch.index_select(self.recv, 0, self.inv_perm, out=self.send)


def _scatter_matrix(g, n_local):
    """0/1 matrix S[n_local, n_send] with S[idx[i], i] = 1, so that ``S @ rows`` is
    ``index_add_(0, idx, rows)`` (aggregator.py:173-175) summed in index order without atomics."""
    m = getattr(g, "_scatter_adj_t", None)
    if m is None:
        idx = g.idx_nodes_send_to_others
        m = SparseTensor(row=idx.cpu(), col=torch.arange(idx.numel()), value=torch.ones(idx.numel()),
                         sparse_sizes=(n_local, idx.numel())).to(idx.device)
        g._scatter_adj_t = m
    return m


def _world_forward(world, feats, bits, out_all=None):
    """The forward data flow for all partitions of ``world`` with the exchange format ``bits`` (32: fp32 rows,
    16: bf16 rows, 8/4/2: packed).  ``out_all`` (optional, [sum n_p, F]) receives the partitions' outputs as
    consecutive row blocks."""
    graphs, pre = world.graphs, world.is_pre_delay
    quantized = bits in (2, 4, 8)
    F = feats[0].shape[-1]
    arena = world.arena(F, feats[0].device, bits)
    qz = Quantizer_for_all_procs(len(graphs), bits) if quantized else None
    fused = quantized and F % 2 == 0
    feats = [x.contiguous() for x in feats]
    main = torch.cuda.current_stream()
    side = world.side_stream(feats[0].device)
    side.wait_stream(main)
    with torch.cuda.stream(side):                                     # send-side chain + exchange
        for g, x in zip(graphs, feats):
            send_buf = g.comm_buf.send_buf
            if not send_buf.shape[0]:
                continue
            q = g.comm_buf_for_quantization
            if pre:
                SPMM_forward(g.adj_t_pre_post_aggr_to, x, send_buf, accumulate=False)   # aggregator.py:41,46
            elif not quantized:
                torch.index_select(x, 0, g.idx_nodes_send_to_others, out=send_buf)   # aggregator.py:48
            if quantized:                                             # communicator.py:269
                qz.quantize_fp32_to_intX(x if not pre else send_buf, q.quantized_send_data_buf, q.send_params,
                                         q.quantized_work_range_per_proc,
                                         row_index=None if pre else g.idx_nodes_send_to_others)
        arena.exchange("forward", quantized)
    outs = []
    row0 = 0
    for g, x in zip(graphs, feats):                                   # overlaps the chain above
        n_p = g.local_adj_t.sparse_size(0)
        out = (out_all[row0:row0 + n_p] if out_all is not None
               else torch.empty((n_p, F), dtype=torch.float32, device=x.device))
        row0 += n_p
        SPMM_forward(g.local_adj_t, x, out, accumulate=False)         # aggregator.py:57,62-65
        outs.append(out)
    main.wait_stream(side)
    for g, out in zip(graphs, outs):
        remote = g.adj_t_pre_post_aggr_from if pre else g.remote_adj_t
        if not remote.sparse_size(1):
            continue
        q = g.comm_buf_for_quantization
        if fused:                                                     # aggregator.py:72-93 in one pass
            SPMM_forward_quantized(remote, q.quantized_recv_data_buf, q.recv_params,
                                   q.dequantized_work_range_per_proc, bits, out)
        else:
            if quantized:
                qz.dequantize_intX_to_fp32(q.quantized_recv_data_buf, g.comm_buf.recv_buf, q.recv_params,
                                           q.dequantized_work_range_per_proc)
            SPMM_forward(remote, g.comm_buf.recv_buf, out)             # aggregator.py:90/92
    return outs


def _world_backward(world, grads, bits, out_all=None):
    """The backward data flow (gradient w.r.t. every partition's node features)."""
    graphs, pre = world.graphs, world.is_pre_delay
    quantized = bits in (2, 4, 8)
    F = grads[0].shape[-1]
    arena = world.arena(F, grads[0].device, bits)
    qz = Quantizer_for_all_procs(len(graphs), bits) if quantized else None
    fused = quantized and F % 2 == 0
    grads = [go.contiguous() for go in grads]
    main = torch.cuda.current_stream()
    side = world.side_stream(grads[0].device)
    side.wait_stream(main)
    with torch.cuda.stream(side):
        for g, go in zip(graphs, grads):
            recv_buf = g.comm_buf.recv_buf
            if not recv_buf.shape[0]:
                continue
            remote = g.adj_t_pre_post_aggr_from if pre else g.remote_adj_t
            SPMM_backward(remote, go, recv_buf, accumulate=False)     # aggregator.py:122,125/127
            if quantized:                                             # the reverse trip is quantized too
                q = g.comm_buf_for_quantization
                qz.quantize_fp32_to_intX(recv_buf, q.quantized_recv_data_buf, q.recv_params,
                                         q.dequantized_work_range_per_proc)
        arena.exchange("backward", quantized)
    outs = []
    row0 = 0
    for g, go in zip(graphs, grads):
        n_p = g.local_adj_t.sparse_size(1)
        local_grad = (out_all[row0:row0 + n_p] if out_all is not None
                      else torch.empty((n_p, F), dtype=torch.float32, device=go.device))
        row0 += n_p
        SPMM_backward(g.local_adj_t, go, local_grad, accumulate=False)   # aggregator.py:140,145-148
        outs.append(local_grad)
    main.wait_stream(side)
    for g, local_grad in zip(graphs, outs):
        send_buf = g.comm_buf.send_buf
        if not send_buf.shape[0]:
            continue
        q = g.comm_buf_for_quantization
        if quantized and not fused:                                   # aggregator.py:159-164
            qz.dequantize_intX_to_fp32(q.quantized_send_data_buf, send_buf, q.send_params,
                                       q.quantized_work_range_per_proc)
        if pre:                                                       # aggregator.py:171
            if fused:
                SPMM_backward_quantized(g.adj_t_pre_post_aggr_to, q.quantized_send_data_buf, q.send_params,
                                        q.quantized_work_range_per_proc, bits, local_grad)
            else:
                SPMM_backward(g.adj_t_pre_post_aggr_to, send_buf, local_grad)
        else:                                                         # aggregator.py:173-175
            scatter = _scatter_matrix(g, local_grad.shape[0])
            if fused:
                SPMM_forward_quantized(scatter, q.quantized_send_data_buf, q.send_params,
                                       q.quantized_work_range_per_proc, bits, local_grad)
            else:
                SPMM_forward(scatter, send_buf, local_grad)
    return outs


class LoopbackAggregator(torch.autograd.Function):
    """``outs = LoopbackAggregator.apply(world, *feats)`` with ``world = LoopbackWorld(...)``;
    ``feats[p]`` are partition p's node features [n_p, F] on the GPU, ``outs[p]`` its aggregated rows."""

    @staticmethod
    def forward(ctx, world, *feats):
        ctx.world = world
        return tuple(_world_forward(world, feats, world.num_bits))

    @staticmethod
    def backward(ctx, *grads):
        return (None,) + tuple(_world_backward(ctx.world, grads, ctx.world.num_bits))


class Aggregator(torch.autograd.Function):
    """``out = Aggregator.apply(graph, local_nodes_feat, layer, num_bits, is_pre_delay, is_training)`` -- the
    reference's autograd Function with the reference's argument list (super_gnn/aggregator.py:15-23, backward
    :96-177), for everything that runs in ONE process on one GPU:

      * ``graph`` a DistributedGraph / DistributedGraphForPre whose partition is the whole graph
        (``world_size == 1`` in the reference: no rows cross a boundary, only ``local_adj_t`` is used,
        aggregator.py:43,62-65,145-148);
      * ``graph`` a LoopbackWorld holding P partitions of one graph: ``local_nodes_feat`` is then the feature
        matrix of all nodes, partition after partition (``world.node_offsets``), and the result has the same row
        order.  The P ranks' steps run one after the other in this process and the all-to-all is the world's
        loop-back exchange; num_bits / is_pre_delay must be the ones the partitions were built for.

    As in the reference, ``is_training == False`` exchanges fp32 rows whatever ``num_bits`` says
    (communicator.py:61-62; the backward pass always uses ``num_bits``), 16 ships bf16 copies of the rows
    (communicator.py:101-127), and ``layer`` only labels timers there (aggregator.py:50): accepted, unused."""

    @staticmethod
    def forward(ctx, graph, local_nodes_feat, layer, num_bits, is_pre_delay, is_training):
        world = _as_world(graph, num_bits, is_pre_delay)
        ctx.world, ctx.num_bits = world, int(num_bits)
        x = local_nodes_feat.contiguous()
        feats = torch.split(x, world.partition_sizes) if len(world.graphs) > 1 else (x,)
        out = torch.empty((world.node_offsets[-1], x.shape[-1]), dtype=torch.float32, device=x.device)
        _world_forward(world, feats, int(num_bits) if is_training else 32, out_all=out)
        return out

    @staticmethod
    def backward(ctx, local_out_grad):
        world = ctx.world
        g = local_out_grad.contiguous()
        grads = torch.split(g, world.partition_sizes) if len(world.graphs) > 1 else (g,)
        out = torch.empty((world.node_offsets[-1], g.shape[-1]), dtype=torch.float32, device=g.device)
        _world_backward(world, grads, ctx.num_bits, out_all=out)
        return None, out, None, None, None, None


def _as_world(graph, num_bits, is_pre_delay):
    if int(num_bits) not in (32, 16, 8, 4, 2):
        raise ValueError(f"num_bits={num_bits}: the exchange formats are 32, 16, 8, 4 and 2")
    if isinstance(graph, LoopbackWorld):
        if graph.is_pre_delay != bool(is_pre_delay):
            raise ValueError("is_pre_delay differs from the mode the world's partitions were built for")
        if int(num_bits) in (2, 4, 8) and graph.num_bits != int(num_bits):
            raise ValueError(f"num_bits={num_bits}, but the world's packed-row splits were built for {graph.num_bits}")
        return graph
    world = getattr(graph, "_sgnn_world", None)
    if world is None or world.is_pre_delay != bool(is_pre_delay):
        from .data_manager import CommBuffer, CommBufferForQuantization, CommSplits
        splits = graph.comm_splits
        if splits is not None and (sum(splits.send_splits) or sum(splits.recv_splits)):
            raise ValueError("this partition exchanges rows with other ranks: put all partitions of the graph into a "
                             "LoopbackWorld and pass that as the graph (one process holds every rank here)")
        dev = graph.local_adj_t.csr()[0].device
        if splits is None or not hasattr(splits, "send_splits_int2"):
            graph.comm_splits = CommSplits([0], [0], 1, 2)      # world_size == 1: nothing crosses a boundary
        if graph.comm_buf is None:
            graph.comm_buf = CommBuffer(graph.comm_splits, 0, 32, device=dev)
        if graph.comm_buf_for_quantization is None:
            graph.comm_buf_for_quantization = CommBufferForQuantization(graph.comm_splits, 0, 2, device=dev)
        world = LoopbackWorld([graph], int(num_bits), bool(is_pre_delay))
        graph._sgnn_world = world
    return world


class LoopbackWorld(object):
    """The P partitions of one graph plus the aggregation settings the reference passes per call
    (num_bits, is_pre_delay).  ``params_wire_dtype=torch.bfloat16`` keeps (zero_point, scale) in the
    reference's bf16 wire format (communicator.py:283-294) from the quantizer to the consumer; None
    keeps them fp32."""

    def __init__(self, graphs: Sequence[object], num_bits: int, is_pre_delay: bool, params_wire_dtype=None) -> None:
        self.graphs = list(graphs)
        self.num_bits = int(num_bits)
        self.is_pre_delay = bool(is_pre_delay)
        if params_wire_dtype not in (None, torch.float32, torch.bfloat16):
            raise ValueError("params_wire_dtype must be None, torch.float32 or torch.bfloat16")
        self.params_wire_dtype = params_wire_dtype
        self._arenas = {}
        self._current = None
        self._side = None
        self._in_degrees = None

    def arena(self, F, device, bits=None):
        """Buffers are kept per feature width and exchange format; the partitions' buffer attributes are
        views of the arena requested last (a layer sequence that alternates widths switches views)."""
        bits = self.num_bits if bits is None else int(bits)
        mode = "q" if bits in (2, 4, 8) else "bf16" if bits == 16 else "fp32"
        a = self._arenas.get((F, mode))
        if a is None:
            a = _Arena(self.graphs, F, mode == "q", self.params_wire_dtype or torch.float32, device, half=mode == "bf16")
            self._arenas[(F, mode)] = a
        if self._current is not a:
            a.bind(self.graphs)
            self._current = a
        return a

    @property
    def partition_sizes(self):
        return [g.local_adj_t.sparse_size(0) for g in self.graphs]

    @property
    def node_offsets(self):
        return _cumulative(self.partition_sizes)

    @property
    def in_degrees(self):
        """[N, 1] in-degrees of all nodes in partition order (what DistSAGEConvGrad divides by, sageconv.py:78)."""
        if self._in_degrees is None:
            self._in_degrees = torch.cat([g.in_degrees.reshape(-1, 1) for g in self.graphs])
        return self._in_degrees

    def side_stream(self, device):
        if self._side is None:
            self._side = torch.cuda.Stream(device=device)   # default priority
        return self._side

    def aggregate(self, feats: Sequence[torch.Tensor]) -> List[torch.Tensor]:
        return list(LoopbackAggregator.apply(self, *feats))
