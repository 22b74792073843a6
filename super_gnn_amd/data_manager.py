"""Per-partition graph objects and communication buffers with the shapes of the reference's
``super_gnn/data_manager`` (CommSplits.py:6-18, CommBuffer.py:5-48, DistributedGraph.py:9-75), plus a
builder that cuts ONE global graph into P vertex partitions inside a single process, so that the
aggregation data flow of ``super_gnn/aggregator.py`` can run on one GPU with a loop-back exchange.

The reference builds these objects per MPI rank from ParMETIS partition files with handshakes between
ranks (DataProcessor.py:17-123, :258-281); here every partition is built from the global CSR directly.
The pre/post-aggregation split uses a simple per-rank-pair vertex cover (all sources or all
destinations of the pair's boundary edges, whichever is fewer) instead of the reference's minimum
vertex cover: any vertex cover yields a correct data flow; only the communication volume differs."""
import math
from typing import List, Optional

import torch
from torch import Tensor

from .sparse import SparseTensor


class CommSplits(object):
    """Rows exchanged with every rank, and the packed rows they occupy when quantized
    (super_gnn/data_manager/CommSplits.py:6-18; the ``_int2`` suffix is the reference's name for any
    bit width)."""

    def __init__(self, recv_splits: list, send_splits: list, world_size: int, bits: int) -> None:
        self.recv_splits = list(recv_splits)
        self.send_splits = list(send_splits)
        if bits in (2, 4, 8):
            per_byte = 8 // bits
            self.recv_splits_int2 = [math.ceil(n / per_byte) for n in self.recv_splits]
            self.send_splits_int2 = [math.ceil(n / per_byte) for n in self.send_splits]


class CommBuffer(object):
    """fp32 message buffers [sum(splits), F] (super_gnn/data_manager/CommBuffer.py:5-27)."""

    def __init__(self, comm_splits: CommSplits, feat_len: int, bits: int, device="cuda") -> None:
        self.send_buf = torch.zeros((sum(comm_splits.send_splits), feat_len), dtype=torch.float32, device=device)
        self.recv_buf = torch.zeros((sum(comm_splits.recv_splits), feat_len), dtype=torch.float32, device=device)

    def resize_buffer(self, comm_splits: CommSplits, feat_len: int, bits: int) -> None:
        for name, n in (("send_buf", sum(comm_splits.send_splits)), ("recv_buf", sum(comm_splits.recv_splits))):
            buf = getattr(self, name)
            if tuple(buf.shape) != (n, feat_len):
                setattr(self, name, torch.zeros((n, feat_len), dtype=torch.float32, device=buf.device))


class CommBufferForQuantization(object):
    """Packed data, per-row params and the cumulative per-rank row ranges
    (super_gnn/data_manager/CommBuffer.py:28-48)."""

    def __init__(self, comm_splits: CommSplits, feat_len: int, bits: int, device="cuda") -> None:
        self.quantized_send_data_buf = torch.zeros((sum(comm_splits.send_splits_int2), feat_len), dtype=torch.uint8, device=device)
        self.quantized_recv_data_buf = torch.zeros((sum(comm_splits.recv_splits_int2), feat_len), dtype=torch.uint8, device=device)
        self.quantized_send_params_buf_fp32 = torch.zeros((sum(comm_splits.send_splits), 2), dtype=torch.float32, device=device)
        self.quantized_recv_params_buf_fp32 = torch.zeros((sum(comm_splits.recv_splits), 2), dtype=torch.float32, device=device)
        self.quantized_work_range_per_proc = torch.zeros(len(comm_splits.send_splits) + 1, dtype=torch.int32)
        self.quantized_work_range_per_proc[1:] = torch.tensor(comm_splits.send_splits, dtype=torch.int32).cumsum(0)
        self.dequantized_work_range_per_proc = torch.zeros(len(comm_splits.recv_splits) + 1, dtype=torch.int32)
        self.dequantized_work_range_per_proc[1:] = torch.tensor(comm_splits.recv_splits, dtype=torch.int32).cumsum(0)

    def resize_buffer(self, comm_splits: CommSplits, feat_len: int, bits: int) -> None:
        for name, n in (("quantized_send_data_buf", sum(comm_splits.send_splits_int2)),
                        ("quantized_recv_data_buf", sum(comm_splits.recv_splits_int2))):
            buf = getattr(self, name)
            if tuple(buf.shape) != (n, feat_len):
                setattr(self, name, torch.zeros((n, feat_len), dtype=torch.uint8, device=buf.device))


class DistributedGraph(object):
    """One partition without pre-aggregation (super_gnn/data_manager/DistributedGraph.py:9-49):
    ``remote_adj_t`` has one column per remote node this partition needs, ordered by owner rank then
    node id; ``idx_nodes_send_to_others`` lists the local nodes other ranks need, ordered by
    destination rank then node id."""

    def __init__(self, local_adj_t: SparseTensor, remote_adj_t: SparseTensor, idx_nodes_send_to_others: Tensor,
                 num_nodes_send_to_others: list, num_nodes_recv_from_others: list, in_degrees: Tensor,
                 comm_splits: CommSplits, comm_buf: Optional[CommBuffer],
                 comm_buf_for_quantization: Optional[CommBufferForQuantization]) -> None:
        self.local_adj_t = local_adj_t
        self.remote_adj_t = remote_adj_t
        self.idx_nodes_send_to_others = idx_nodes_send_to_others
        self.num_nodes_send_to_others = num_nodes_send_to_others
        self.num_nodes_recv_from_others = num_nodes_recv_from_others
        self.in_degrees = in_degrees
        self.comm_splits = comm_splits
        self.comm_buf = comm_buf
        self.comm_buf_for_quantization = comm_buf_for_quantization


class DistributedGraphForPre(object):
    """One partition with pre/post aggregation (super_gnn/data_manager/DistributedGraph.py:51-75):
    ``send_buf = adj_t_pre_post_aggr_to @ local_feat`` and ``out += adj_t_pre_post_aggr_from @ recv_buf``."""

    def __init__(self, local_adj_t: SparseTensor, adj_t_pre_post_aggr_from: SparseTensor,
                 adj_t_pre_post_aggr_to: SparseTensor, pre_post_aggr_from_splits: list, pre_post_aggr_to_splits: list,
                 in_degrees: Tensor, comm_splits: CommSplits, comm_buf: Optional[CommBuffer],
                 comm_buf_for_quantization: Optional[CommBufferForQuantization]) -> None:
        self.local_adj_t = local_adj_t
        self.adj_t_pre_post_aggr_from = adj_t_pre_post_aggr_from
        self.adj_t_pre_post_aggr_to = adj_t_pre_post_aggr_to
        self.pre_post_aggr_from_splits = pre_post_aggr_from_splits
        self.pre_post_aggr_to_splits = pre_post_aggr_to_splits
        self.in_degrees = in_degrees
        self.comm_splits = comm_splits
        self.comm_buf = comm_buf
        self.comm_buf_for_quantization = comm_buf_for_quantization


def _coo_to_sparse(row, col, val, sizes, device):
    return SparseTensor(row=row, col=col, value=val, sparse_sizes=sizes).to(device)


def build_loopback_partitions(rowptr: Tensor, col: Tensor, value: Optional[Tensor], num_parts: int, feat_len: int,
                              num_bits: int = 32, is_pre_delay: bool = False, device="cuda") -> List[object]:
    """Cut the global graph (CSR over destination rows, i.e. the transposed adjacency the reference
    calls ``adj_t``) into ``num_parts`` contiguous vertex ranges and build each partition's graph
    object, comm splits and buffers.  Returns a list of DistributedGraph / DistributedGraphForPre,
    each with an extra attribute ``node_range = (begin, end)``."""
    rowptr = rowptr.detach().cpu().to(torch.int64)
    col = col.detach().cpu().to(torch.int64)
    N = rowptr.numel() - 1
    P = int(num_parts)
    val = value.detach().cpu().to(torch.float32) if value is not None else torch.ones(col.numel())
    bounds = torch.tensor([N * p // P for p in range(P + 1)], dtype=torch.int64)
    deg = rowptr[1:] - rowptr[:-1]
    row = torch.repeat_interleave(torch.arange(N), deg)
    owner_of = lambda ids: torch.searchsorted(bounds, ids, right=True) - 1  # noqa: E731

    # per destination partition r: local edges and remote edges grouped by source owner
    parts = []
    for r in range(P):
        b, e = int(bounds[r]), int(bounds[r + 1])
        sel = slice(int(rowptr[b]), int(rowptr[e]))
        rr, cc, ww = row[sel] - b, col[sel], val[sel]
        is_local = (cc >= b) & (cc < e)
        parts.append({"range": (b, e), "n": e - b,
                      "local": (rr[is_local], cc[is_local] - b, ww[is_local]),
                      "remote": (rr[~is_local], cc[~is_local], ww[~is_local])})

    # boundary blocks: blocks[p][r] = (rows (rows at the receiver r), cols (source nodes local to p), weights)
    seg_rows = [[0] * P for _ in range(P)]          # rows exchanged p -> r
    to_blocks = [[None] * P for _ in range(P)]      # at the sender p: (seg_row, local_src, w)
    from_blocks = [[None] * P for _ in range(P)]    # at the receiver r: (local_dst, seg_row, w)
    send_idx = [[None] * P for _ in range(P)]       # non-pre mode: local nodes of p that r needs
    for r in range(P):
        v, u_glob, w = parts[r]["remote"]
        own = owner_of(u_glob)
        for p in range(P):
            if p == r:
                continue
            m = own == p
            if not bool(m.any()):
                continue
            vv, uu, wwp = v[m], u_glob[m] - int(bounds[p]), w[m]
            src_nodes, src_inv = torch.unique(uu, return_inverse=True)
            dst_nodes, dst_inv = torch.unique(vv, return_inverse=True)
            if not is_pre_delay or src_nodes.numel() <= dst_nodes.numel():
                # post-aggregation: ship the source rows, apply the edges at the receiver
                n = src_nodes.numel()
                to_blocks[p][r] = (torch.arange(n), src_nodes, torch.ones(n))
                from_blocks[p][r] = (vv, src_inv, wwp)
                send_idx[p][r] = src_nodes
            else:
                # pre-aggregation: ship one partial sum per destination node
                n = dst_nodes.numel()
                to_blocks[p][r] = (dst_inv, uu, wwp)
                from_blocks[p][r] = (dst_nodes, torch.arange(n), torch.ones(n))
            seg_rows[p][r] = n

    graphs = []
    for r in range(P):
        n_r = parts[r]["n"]
        send_splits = [seg_rows[r][d] for d in range(P)]
        recv_splits = [seg_rows[s][r] for s in range(P)]
        lr, lc, lw = parts[r]["local"]
        local_adj_t = _coo_to_sparse(lr, lc, lw, (n_r, n_r), device)
        # receive side: columns = concatenated segments from every source rank
        fr, fc, fw, off = [], [], [], 0
        for s in range(P):
            if from_blocks[s][r] is not None:
                a, bcol, w = from_blocks[s][r]
                fr.append(a); fc.append(bcol + off); fw.append(w)
            off += recv_splits[s]
        cat = lambda xs, dt: torch.cat(xs) if xs else torch.empty(0, dtype=dt)  # noqa: E731
        adj_from = _coo_to_sparse(cat(fr, torch.int64), cat(fc, torch.int64), cat(fw, torch.float32), (n_r, off), device)
        # send side: rows = concatenated segments for every destination rank
        tr, tc, tw, off = [], [], [], 0
        for d in range(P):
            if to_blocks[r][d] is not None:
                a, bcol, w = to_blocks[r][d]
                tr.append(a + off); tc.append(bcol); tw.append(w)
            off += send_splits[d]
        adj_to = _coo_to_sparse(cat(tr, torch.int64), cat(tc, torch.int64), cat(tw, torch.float32), (off, n_r), device)
        in_deg = torch.zeros(n_r)
        in_deg.index_add_(0, lr, torch.ones(lr.numel()))
        rv = parts[r]["remote"][0]
        in_deg.index_add_(0, rv, torch.ones(rv.numel()))
        in_deg = in_deg.clamp(min=1).unsqueeze(-1).to(device)  # DataProcessor.get_in_degrees (:17-23)
        splits = CommSplits(recv_splits, send_splits, P, num_bits)
        buf = CommBuffer(splits, feat_len, num_bits, device)
        qbuf = CommBufferForQuantization(splits, feat_len, num_bits, device) if num_bits in (2, 4, 8) else None
        if is_pre_delay:
            g = DistributedGraphForPre(local_adj_t, adj_from, adj_to, recv_splits, send_splits, in_deg, splits, buf, qbuf)
        else:
            idx = cat([send_idx[r][d] for d in range(P) if send_idx[r][d] is not None], torch.int64).to(device)
            g = DistributedGraph(local_adj_t, adj_from, idx, send_splits, recv_splits, in_deg, splits, buf, qbuf)
        g.node_range = parts[r]["range"]
        graphs.append(g)
    return graphs
