"""Per-partition graph objects and communication buffers with the shapes of the reference's
``super_gnn/data_manager`` (CommSplits.py:6-18, CommBuffer.py:5-48, DistributedGraph.py:9-75), plus a
builder that cuts ONE global graph into P vertex partitions inside a single process, so that the
aggregation data flow of ``super_gnn/aggregator.py`` can run on one GPU with a loop-back exchange.

The reference builds these objects per MPI rank from ParMETIS partition files with handshakes between
ranks (DataLoader.py:17-278, DataProcessor.py:17-541); here every partition is built from the global
CSR directly, and ``load_loopback_partitions`` reads the reference's per-rank files back into that
global CSR first.  The pre/post-aggregation split follows the reference: per ordered rank pair a
minimum vertex cover of the pair's bipartite boundary graph decides, edge by edge, whether the source
row is shipped (source in the cover: post-aggregation at the receiver) or a partial sum per
destination is (pre-aggregation at the sender) (DataProcessor.py:266-289, VertexCoverFinder.py:686-753);
the cover comes from a Hopcroft-Karp maximum matching plus Koenig's construction."""
import math
import os
from typing import List, Optional

import numpy as np
import scipy.sparse as sp
import torch
from scipy.sparse.csgraph import maximum_bipartite_matching
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
    """fp32 message buffers [sum(splits), F], plus bf16 copies of them in the 16-bit exchange mode (the
    reference's attribute names say fp16, the dtype is bfloat16: super_gnn/data_manager/CommBuffer.py:5-27)."""

    def __init__(self, comm_splits: CommSplits, feat_len: int, bits: int, device="cuda") -> None:
        self.send_buf = torch.zeros((sum(comm_splits.send_splits), feat_len), dtype=torch.float32, device=device)
        self.recv_buf = torch.zeros((sum(comm_splits.recv_splits), feat_len), dtype=torch.float32, device=device)
        self.send_buf_fp16 = None
        self.recv_buf_fp16 = None
        if bits == 16:
            self.send_buf_fp16 = torch.zeros_like(self.send_buf, dtype=torch.bfloat16)
            self.recv_buf_fp16 = torch.zeros_like(self.recv_buf, dtype=torch.bfloat16)

    def resize_buffer(self, comm_splits: CommSplits, feat_len: int, bits: int) -> None:
        sizes = (("send_buf", sum(comm_splits.send_splits)), ("recv_buf", sum(comm_splits.recv_splits)))
        for name, n in sizes:
            buf = getattr(self, name)
            if tuple(buf.shape) != (n, feat_len):
                setattr(self, name, torch.zeros((n, feat_len), dtype=torch.float32, device=buf.device))
        if bits == 16 and self.send_buf_fp16 is not None and self.recv_buf_fp16 is not None:
            for name, n in sizes:
                buf = getattr(self, name + "_fp16")
                if tuple(buf.shape) != (n, feat_len):
                    setattr(self, name + "_fp16", torch.zeros((n, feat_len), dtype=torch.bfloat16, device=buf.device))


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


def minimum_vertex_cover(src: np.ndarray, dst: np.ndarray):
    """Minimum vertex cover of the bipartite graph with edges (src[i], dst[i]); sources and
    destinations are separate id spaces.  Returns boolean masks (src_in_cover, dst_in_cover) over the
    *edges' endpoints*: every edge has src_in_cover[i] or dst_in_cover[i], and the number of distinct
    covered endpoints equals the size of a maximum matching (Koenig's theorem).  Same role as
    VertexCoverFinder.find_minimum_vertex_cover (super_gnn/data_manager/VertexCoverFinder.py:697-753)."""
    if src.size == 0:
        return np.zeros(0, bool), np.zeros(0, bool)
    us, ui = np.unique(src, return_inverse=True)
    vs, vi = np.unique(dst, return_inverse=True)
    nu, nv = us.size, vs.size
    g = sp.csr_matrix((np.ones(src.size, np.int8), (ui, vi)), shape=(nu, nv))
    g.sum_duplicates()
    match_u = maximum_bipartite_matching(g, perm_type="column")      # for each u: matched v or -1
    match_v = np.full(nv, -1, np.int64)
    match_v[match_u[match_u >= 0]] = np.nonzero(match_u >= 0)[0]
    # Z = vertices reachable from unmatched u by alternating paths (free edge u->v, matched edge v->u)
    zu = match_u < 0
    zv = np.zeros(nv, bool)
    frontier = np.nonzero(zu)[0]
    indptr, indices = g.indptr, g.indices
    while frontier.size:
        counts = indptr[frontier + 1] - indptr[frontier]
        starts = np.repeat(indptr[frontier], counts)
        offs = np.arange(counts.sum()) - np.repeat(np.cumsum(counts) - counts, counts)
        nbr = np.unique(indices[starts + offs])
        nbr = nbr[~zv[nbr]]
        zv[nbr] = True
        nxt = match_v[nbr]
        nxt = nxt[nxt >= 0]
        nxt = nxt[~zu[nxt]]
        zu[nxt] = True
        frontier = nxt
    cover_u, cover_v = ~zu, zv                                        # (U \ Z) + (V & Z)
    return cover_u[ui], cover_v[vi]


def build_loopback_partitions(rowptr: Tensor, col: Tensor, value: Optional[Tensor], num_parts: int, feat_len: int,
                              num_bits: int = 32, is_pre_delay: bool = False, device="cuda",
                              bounds: Optional[Tensor] = None, cover: str = "minimum") -> List[object]:
    """Cut the global graph (CSR over destination rows, i.e. the transposed adjacency the reference
    calls ``adj_t``) into ``num_parts`` contiguous vertex ranges (``bounds``: the reference's
    begin_node_on_each_partition, default equal ranges) and build each partition's graph object, comm
    splits and buffers.  Returns a list of DistributedGraph / DistributedGraphForPre, each with an
    extra attribute ``node_range = (begin, end)``.

    ``cover`` (pre/post mode only): "minimum" = minimum vertex cover per rank pair (the reference's
    rule), "side" = all sources or all destinations of the pair, whichever is fewer.  Within a segment
    the message rows are ordered by the global id of the node they stand for, as in the reference
    (DataProcessor.py:306-318)."""
    rowptr = rowptr.detach().cpu().to(torch.int64)
    col = col.detach().cpu().to(torch.int64)
    N = rowptr.numel() - 1
    P = int(num_parts)
    val = value.detach().cpu().to(torch.float32) if value is not None else torch.ones(col.numel())
    if bounds is None:
        bounds = torch.tensor([N * p // P for p in range(P + 1)], dtype=torch.int64)
    else:
        bounds = torch.as_tensor(bounds, dtype=torch.int64)
        if bounds.numel() != P + 1 or int(bounds[0]) != 0 or int(bounds[-1]) != N or bool((bounds[1:] < bounds[:-1]).any()):
            raise ValueError("bounds must be P + 1 non-decreasing node offsets from 0 to the node count")
    if cover not in ("minimum", "side"):
        raise ValueError("cover must be 'minimum' or 'side'")
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

    # boundary blocks per ordered pair p -> r (p owns the sources, r the destinations)
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
            vv, uu, wwp = v[m], u_glob[m] - int(bounds[p]), w[m]     # dst local to r, src local to p
            if not is_pre_delay:
                post = torch.ones(vv.numel(), dtype=torch.bool)
            elif cover == "side":
                n_src, n_dst = torch.unique(uu).numel(), torch.unique(vv).numel()
                post = torch.full((vv.numel(),), n_src <= n_dst, dtype=torch.bool)
            else:
                src_in_cover, _ = minimum_vertex_cover(uu.numpy(), vv.numpy())
                post = torch.from_numpy(src_in_cover)                 # DataProcessor.py:283-287
            # message rows: one per shipped source node (post) and one per pre-aggregated destination,
            # ordered by global id (sources of p and destinations of r live in disjoint id ranges)
            post_nodes = torch.unique(uu[post]) + int(bounds[p])
            pre_nodes = torch.unique(vv[~post]) + int(bounds[r])
            keys = torch.cat([post_nodes, pre_nodes])
            order = torch.argsort(keys)
            slot_of = torch.empty_like(order)
            slot_of[order] = torch.arange(order.numel())
            post_slot, pre_slot = slot_of[:post_nodes.numel()], slot_of[post_nodes.numel():]
            e_post_slot = post_slot[torch.searchsorted(post_nodes, uu[post] + int(bounds[p]))]
            e_pre_slot = pre_slot[torch.searchsorted(pre_nodes, vv[~post] + int(bounds[r]))]
            n_post, n_pre = post_nodes.numel(), pre_nodes.numel()
            to_blocks[p][r] = (torch.cat([post_slot, e_pre_slot]),
                               torch.cat([post_nodes - int(bounds[p]), uu[~post]]),
                               torch.cat([torch.ones(n_post), wwp[~post]]))
            from_blocks[p][r] = (torch.cat([vv[post], pre_nodes - int(bounds[r])]),
                                 torch.cat([e_post_slot, pre_slot]),
                                 torch.cat([wwp[post], torch.ones(n_pre)]))
            if not is_pre_delay:
                send_idx[p][r] = post_nodes - int(bounds[p])
            seg_rows[p][r] = n_post + n_pre

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


# ------------------------------------------------------------------------------------------------
# The reference's on-disk partition format (one set of files per rank, written by its
# graph_partition scripts and read by super_gnn/data_manager/DataLoader.py:17-68)
# ------------------------------------------------------------------------------------------------
def _rank_file(input_dir, graph_name, rank, what):
    return os.path.join(input_dir, "p{:0>3d}-{}_{}.npy".format(rank, graph_name, what))


def load_graph_structures(input_dir, graph_name, rank):
    """(local_nodes_list [n,>=1] with the global id in column 0, local_edges_list [2,E] = (src, dst)
    both local ids, remote_edges_list [2,E'] = (global src id, local dst id),
    begin_node_on_each_partition [P+1], num_local_nodes) -- DataLoader.py:17-46."""
    nodes = np.load(_rank_file(input_dir, graph_name, rank, "nodes"))
    local_edges = np.load(_rank_file(input_dir, graph_name, rank, "local_edges"))
    remote_edges = np.load(_rank_file(input_dir, graph_name, rank, "remote_edges"))
    begins = np.loadtxt(os.path.join(input_dir, "begin_node_on_each_partition.txt"), dtype=np.int64, delimiter=" ")
    num_local = int(nodes[-1][0] - nodes[0][0] + 1)
    return (torch.from_numpy(nodes), torch.from_numpy(local_edges), torch.from_numpy(remote_edges),
            torch.from_numpy(np.atleast_1d(begins)), num_local)


def load_nodes_labels(input_dir, graph_name, rank):
    return torch.from_numpy(np.load(_rank_file(input_dir, graph_name, rank, "nodes_label")))   # DataLoader.py:49-54


def load_nodes_features(input_dir, graph_name, rank):
    feat = np.load(_rank_file(input_dir, graph_name, rank, "nodes_feat"))                      # DataLoader.py:57-62
    if feat.dtype == np.float16:
        feat = feat.astype(np.float32)
    return torch.from_numpy(feat)


def load_dataset_mask(input_dir, graph_name, rank):
    return tuple(torch.from_numpy(np.load(_rank_file(input_dir, graph_name, rank, "nodes_%s_idx" % k)))
                 for k in ("train", "valid", "test"))                                        # DataLoader.py:65-68


def load_loopback_partitions(input_dir, graph_name, world_size, feat_len, num_bits=32, is_pre_delay=False,
                             device="cuda", cover="minimum"):
    """Read every rank's files and build the P partitions in this process.  Returns
    (graphs, data) where data[p] is the dict the reference's load_data returns per rank
    (DataLoader.py:213-278): nodes_features, nodes_labels, nodes_{train,valid,test}_masks, plus graph.
    Edge weights are ones, as in DataProcessor.transform_edge_index_to_sparse_tensor (:108-123)."""
    P = int(world_size)
    srcs, dsts, begins = [], [], None
    for rank in range(P):
        nodes, local_edges, remote_edges, b, n_local = load_graph_structures(input_dir, graph_name, rank)
        if begins is None:
            begins = b.to(torch.int64)
            if begins.numel() != P + 1:
                raise ValueError("begin_node_on_each_partition.txt lists %d ranges, world_size is %d" % (begins.numel() - 1, P))
        first = int(nodes[0][0])
        if first != int(begins[rank]) or n_local != int(begins[rank + 1] - begins[rank]):
            raise ValueError("rank %d: node list does not match begin_node_on_each_partition.txt" % rank)
        srcs += [local_edges[0].to(torch.int64) + first, remote_edges[0].to(torch.int64)]
        dsts += [local_edges[1].to(torch.int64) + first, remote_edges[1].to(torch.int64) + first]
    src, dst = torch.cat(srcs), torch.cat(dsts)
    N = int(begins[-1])
    order = torch.argsort(dst * N + src)                 # CSR over destinations, columns ascending
    src, dst = src[order], dst[order]
    rowptr = torch.zeros(N + 1, dtype=torch.int64)
    rowptr[1:] = torch.cumsum(torch.bincount(dst, minlength=N), 0)
    graphs = build_loopback_partitions(rowptr, src, None, P, feat_len, num_bits=num_bits, is_pre_delay=is_pre_delay,
                                       device=device, bounds=begins, cover=cover)
    data = []
    for rank, g in enumerate(graphs):
        train, valid, test = load_dataset_mask(input_dir, graph_name, rank)
        data.append({"graph": g, "nodes_features": load_nodes_features(input_dir, graph_name, rank),
                     "nodes_labels": load_nodes_labels(input_dir, graph_name, rank),
                     "nodes_train_masks": train, "nodes_valid_masks": valid, "nodes_test_masks": test})
    return graphs, data


def save_partition_files(output_dir, graph_name, rowptr, col, bounds, feat, label, train_idx, valid_idx, test_idx):
    """Write a global graph (CSR over destinations) as the reference's per-rank files, for the given
    contiguous node ranges: the layout load_graph_structures reads.  train/valid/test_idx are global
    node ids; each rank stores its own, localized."""
    os.makedirs(output_dir, exist_ok=True)
    rowptr = torch.as_tensor(rowptr, dtype=torch.int64).cpu()
    col = torch.as_tensor(col, dtype=torch.int64).cpu()
    bounds = torch.as_tensor(bounds, dtype=torch.int64).cpu()
    N = rowptr.numel() - 1
    row = torch.repeat_interleave(torch.arange(N), rowptr[1:] - rowptr[:-1])
    np.savetxt(os.path.join(output_dir, "begin_node_on_each_partition.txt"), bounds.numpy()[None, :], fmt="%d", delimiter=" ")
    for rank in range(bounds.numel() - 1):
        b, e = int(bounds[rank]), int(bounds[rank + 1])
        sel = slice(int(rowptr[b]), int(rowptr[e]))
        src, dst = col[sel], row[sel] - b
        local = (src >= b) & (src < e)
        ids = torch.arange(b, e)
        np.save(_rank_file(output_dir, graph_name, rank, "nodes"), torch.stack([ids, ids - b], 1).numpy())
        np.save(_rank_file(output_dir, graph_name, rank, "local_edges"), torch.stack([src[local] - b, dst[local]]).numpy())
        np.save(_rank_file(output_dir, graph_name, rank, "remote_edges"), torch.stack([src[~local], dst[~local]]).numpy())
        np.save(_rank_file(output_dir, graph_name, rank, "nodes_feat"), torch.as_tensor(feat)[b:e].cpu().numpy())
        np.save(_rank_file(output_dir, graph_name, rank, "nodes_label"), torch.as_tensor(label)[b:e].cpu().numpy())
        for name, idx in (("train", train_idx), ("valid", valid_idx), ("test", test_idx)):
            idx = torch.as_tensor(idx, dtype=torch.int64).cpu()
            np.save(_rank_file(output_dir, graph_name, rank, "nodes_%s_idx" % name), (idx[(idx >= b) & (idx < e)] - b).numpy())
