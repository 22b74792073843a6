"""The aggregation data flow of super_gnn/aggregator.py on one GPU: P partitions of one graph in one
process, loop-back exchange.

  * fp32 exchange: the concatenated partition outputs must equal the GLOBAL product A @ X of the
    unpartitioned graph (CPU oracle), forward, and A^T @ G backward -- this pins the partition
    builder, the splits and both exchange directions against something that knows nothing of them;
  * int8/int4/int2 exchange: must equal the same flow computed on the CPU with the oracle's
    quantize -> dequantize at every boundary crossing."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from oracle import oracle as orc
from _util import abs_sum64, assert_spmm_close

pytestmark = pytest.mark.gpu


def _graph(n=12000, und_edges=90000, seed=5):
    from super_gnn_amd import synth
    rowptr, col = synth.rmat_graph(n, und_edges, seed=seed)
    w = synth.gcn_norm_weights(rowptr, col)
    return rowptr, col, w


def _csr_np(st):
    rowptr, col, val = st.csr()
    return rowptr.cpu().numpy().astype(np.int64), col.cpu().numpy().astype(np.int64), val.cpu().numpy().astype(np.float32)


def _cpu_spmm(st, x, out):
    rp, c, v = _csr_np(st)
    if out.shape[0]:
        orc.spmm_accumulate(rp, c, v, np.ascontiguousarray(x), out)


@pytest.mark.parametrize("pre", [False, True])
@pytest.mark.parametrize("P", [1, 4])
def test_fp32_exchange_equals_global_product(pre, P):
    from super_gnn_amd.aggregator import LoopbackWorld
    from super_gnn_amd.data_manager import build_loopback_partitions
    rowptr, col, w = _graph()
    n, F = rowptr.numel() - 1, 64
    graphs = build_loopback_partitions(rowptr, col, w, P, F, num_bits=32, is_pre_delay=pre)
    assert sum(g.local_adj_t.sparse_size(0) for g in graphs) == n
    for g in graphs:  # every send segment is mirrored by the peer's recv segment
        for r, h in enumerate(graphs):
            assert g.comm_splits.send_splits[r] == h.comm_splits.recv_splits[graphs.index(g)]
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n, F, generator=gen)
    feats = [x[g.node_range[0]:g.node_range[1]].cuda().requires_grad_() for g in graphs]
    world = LoopbackWorld(graphs, 32, pre)
    outs = world.aggregate(feats)
    got = torch.cat(outs).detach().cpu().numpy()
    rp, c, v = rowptr.numpy(), col.numpy().astype(np.int64), w.numpy()
    want = np.zeros((n, F), np.float32)
    orc.spmm_accumulate(rp, c, v, x.numpy(), want)
    assert_spmm_close(got, want, orc.spmm_f64(rp, c, v, x.numpy()), abs_sum64(rp, c, v, x.numpy()), np.diff(rp), what="forward")
    # backward: d(sum(out * G))/dX = A^T G
    G = torch.randn(n, F, generator=gen)
    torch.autograd.backward(outs, [G[g.node_range[0]:g.node_range[1]].cuda() for g in graphs])
    got_g = torch.cat([f.grad for f in feats]).cpu().numpy()
    AT = sp.csr_matrix((v, c, rp), shape=(n, n)).T.tocsr(); AT.sort_indices()
    rpt, ct, vt = AT.indptr.astype(np.int64), AT.indices.astype(np.int64), AT.data.astype(np.float32)
    want_g = np.zeros((n, F), np.float32)
    orc.spmm_accumulate(rpt, ct, vt, G.numpy(), want_g)
    assert_spmm_close(got_g, want_g, orc.spmm_f64(rpt, ct, vt, G.numpy()), abs_sum64(rpt, ct, vt, G.numpy()), np.diff(rpt), what="backward")
    if pre and P > 1:  # pre-aggregation must not send more rows than plain boundary exchange would
        plain = build_loopback_partitions(rowptr, col, w, P, F, num_bits=32, is_pre_delay=False)
        assert sum(sum(g.comm_splits.send_splits) for g in graphs) <= sum(sum(g.comm_splits.send_splits) for g in plain)


@pytest.mark.parametrize("bits", [8, 4, 2])
@pytest.mark.parametrize("pre", [False, True])
def test_quantized_exchange_equals_cpu_flow(bits, pre):
    from super_gnn_amd.aggregator import LoopbackWorld
    from super_gnn_amd.data_manager import build_loopback_partitions
    rowptr, col, w = _graph(n=8000, und_edges=60000, seed=9)
    n, F, P = rowptr.numel() - 1, 128, 4
    graphs = build_loopback_partitions(rowptr, col, w, P, F, num_bits=bits, is_pre_delay=pre)
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(n, F, generator=gen)
    xs = [x[g.node_range[0]:g.node_range[1]] for g in graphs]
    feats = [t.cuda().requires_grad_() for t in xs]
    outs = LoopbackWorld(graphs, bits, pre).aggregate(feats)

    def crossing(buf, splits):
        """what a buffer looks like on the far side: quantize per segment, dequantize (oracle)"""
        seg = np.concatenate([[0], np.cumsum(splits)]).astype(np.int32)
        if buf.shape[0] == 0:
            return buf
        q, prm = orc.quant_rows(np.ascontiguousarray(buf), seg, bits)
        return orc.dequant_rows(q, prm, seg, bits, buf.shape[1])

    # forward on the CPU
    sent = []
    for g, xp in zip(graphs, xs):
        ns = sum(g.comm_splits.send_splits)
        sb = np.zeros((ns, F), np.float32)
        if pre:
            _cpu_spmm(g.adj_t_pre_post_aggr_to, xp.numpy(), sb)
        elif ns:
            sb = xp.numpy()[g.idx_nodes_send_to_others.cpu().numpy()]
        sent.append(crossing(sb, g.comm_splits.send_splits))
    want_outs = []
    for r, (g, xp) in enumerate(zip(graphs, xs)):
        segs = []
        for p, h in enumerate(graphs):
            o = np.concatenate([[0], np.cumsum(h.comm_splits.send_splits)])
            segs.append(sent[p][o[r]:o[r + 1]])
        recv = np.concatenate(segs) if segs else np.zeros((0, F), np.float32)
        out = np.zeros((g.local_adj_t.sparse_size(0), F), np.float32)
        _cpu_spmm(g.local_adj_t, xp.numpy(), out)
        _cpu_spmm(g.adj_t_pre_post_aggr_from if pre else g.remote_adj_t, recv, out)
        want_outs.append(out)
    for r, (o, wnt) in enumerate(zip(outs, want_outs)):
        got = o.detach().cpu().numpy()
        assert np.all(np.abs(got - wnt) <= 1e-4 + 1e-4 * np.abs(wnt)), f"rank {r}"  # hub rows: summation order
        assert (np.abs(got - wnt) <= 1e-6 + 1e-5 * np.abs(wnt)).mean() > 0.999
    # backward runs, is finite, and is close to the unquantized gradient at the quantization error scale
    G = torch.randn(n, F, generator=gen)
    torch.autograd.backward(outs, [G[g.node_range[0]:g.node_range[1]].cuda() for g in graphs])
    got_g = torch.cat([f.grad for f in feats]).cpu().numpy()
    rp, c, v = rowptr.numpy(), col.numpy().astype(np.int64), w.numpy()
    AT = sp.csr_matrix((v, c, rp), shape=(n, n)).T.tocsr()
    exact_g = AT @ G.numpy()
    assert np.isfinite(got_g).all()
    rel = np.linalg.norm(got_g - exact_g) / np.linalg.norm(exact_g)
    assert rel < {8: 0.01, 4: 0.1, 2: 0.5}[bits], rel


@pytest.mark.parametrize("bits,pre", [(8, False), (2, False), (4, True), (2, True)])
def test_bf16_param_transport_matches_reference_wire_format(bits, pre):
    """With bf16 params the world must give exactly the floats of the reference's sequence
    (communicator.py:269-294, aggregator.py:72-93): quantize with fp32 params, copy_ to bf16, move,
    copy_ back to fp32, dequantize, SpMM -- rebuilt here from the unfused GPU operators."""
    from super_gnn_amd import Quantizer_for_all_procs, SPMM_forward
    from super_gnn_amd.aggregator import LoopbackWorld
    from super_gnn_amd.data_manager import build_loopback_partitions
    rowptr, col, w = _graph(n=4000, und_edges=30000, seed=2)
    n, F, P = rowptr.numel() - 1, 64, 3
    graphs = build_loopback_partitions(rowptr, col, w, P, F, num_bits=bits, is_pre_delay=pre)
    x = torch.randn(n, F, generator=torch.Generator().manual_seed(3))
    feats = [x[g.node_range[0]:g.node_range[1]].cuda() for g in graphs]
    o32 = LoopbackWorld(graphs, bits, pre).aggregate(feats)
    world16 = LoopbackWorld(graphs, bits, pre, params_wire_dtype=torch.bfloat16)
    o16 = world16.aggregate(feats)
    prm = graphs[0].comm_buf_for_quantization.quantized_recv_params_buf_bf16
    assert prm.dtype == torch.bfloat16 and prm.shape[0] == sum(graphs[0].comm_splits.recv_splits)

    qz = Quantizer_for_all_procs(P, bits)
    crossed = []   # per sender: its send rows after quantize -> bf16 params -> dequantize
    for g, xp in zip(graphs, feats):
        ns = sum(g.comm_splits.send_splits)
        sb = torch.zeros((ns, F), device="cuda")
        if pre:
            SPMM_forward(g.adj_t_pre_post_aggr_to, xp, sb)
        elif ns:
            sb = xp[g.idx_nodes_send_to_others].contiguous()
        wr = torch.tensor([0] + list(np.cumsum(g.comm_splits.send_splits)), dtype=torch.int32)
        q = torch.zeros((sum(g.comm_splits.send_splits_int2), F), dtype=torch.uint8, device="cuda")
        p32 = torch.zeros((ns, 2), device="cuda")
        back = torch.zeros_like(sb)
        if ns:
            qz.quantize_fp32_to_intX(sb, q, p32, wr)
            p_wire = p32.to(torch.bfloat16).to(torch.float32)
            qz.dequantize_intX_to_fp32(q, back, p_wire, wr)
        crossed.append(back)
    for r, (g, xp) in enumerate(zip(graphs, feats)):
        segs = []
        for p, h in enumerate(graphs):
            o = np.concatenate([[0], np.cumsum(h.comm_splits.send_splits)])
            segs.append(crossed[p][o[r]:o[r + 1]])
        recv = torch.cat(segs).contiguous()
        out = torch.zeros((g.local_adj_t.sparse_size(0), F), device="cuda")
        SPMM_forward(g.local_adj_t, xp, out)
        if recv.shape[0]:
            SPMM_forward(g.adj_t_pre_post_aggr_from if pre else g.remote_adj_t, recv, out)
        assert torch.equal(out, o16[r]), f"rank {r}"
    a, b = torch.cat(o32), torch.cat(o16)
    assert not torch.equal(a, b) and torch.allclose(a, b, atol=0.1, rtol=0.1)


def test_backward_is_deterministic_and_matches_unfused_scatter():
    """Plain mode, int8: the fused dequantize+scatter of the returned gradient rows equals
    dequantize followed by a sequential index_add (reference: aggregator.py:159-175), run to run."""
    from super_gnn_amd.aggregator import LoopbackWorld
    from super_gnn_amd.data_manager import build_loopback_partitions
    rowptr, col, w = _graph(n=5000, und_edges=40000, seed=12)
    n, F, P = rowptr.numel() - 1, 32, 4
    graphs = build_loopback_partitions(rowptr, col, w, P, F, num_bits=8, is_pre_delay=False)
    gen = torch.Generator().manual_seed(5)
    x, G = torch.randn(n, F, generator=gen), torch.randn(n, F, generator=gen)
    world = LoopbackWorld(graphs, 8, False)
    runs = []
    for _ in range(2):
        feats = [x[g.node_range[0]:g.node_range[1]].cuda().requires_grad_() for g in graphs]
        outs = world.aggregate(feats)
        torch.autograd.backward(outs, [G[g.node_range[0]:g.node_range[1]].cuda() for g in graphs])
        runs.append(torch.cat([f.grad for f in feats]))
    assert torch.equal(runs[0], runs[1])
    # rebuild partition 0's gradient from what the exchange left in its buffers
    from super_gnn_amd import Quantizer_for_all_procs, SPMM_backward
    g = graphs[0]
    q = g.comm_buf_for_quantization
    rows = torch.zeros_like(g.comm_buf.send_buf)
    Quantizer_for_all_procs(P, 8).dequantize_intX_to_fp32(q.quantized_send_data_buf, rows, q.send_params,
                                                          q.quantized_work_range_per_proc)
    want = torch.zeros((g.node_range[1] - g.node_range[0], F), device="cuda")
    SPMM_backward(g.local_adj_t, G[g.node_range[0]:g.node_range[1]].cuda(), want)
    want = want.cpu()
    for i, node in enumerate(g.idx_nodes_send_to_others.cpu().tolist()):   # index order, one add per row
        want[node] += rows[i].cpu()
    assert torch.equal(runs[0][:want.shape[0]].cpu(), want)


def test_sage_model_is_partition_invariant_and_trains():
    """A 3-layer GraphSAGE over 4 partitions (fp32 exchange) must produce the outputs and weight
    gradients of the same model over the unpartitioned graph; with an int2 exchange it must still train."""
    from super_gnn_amd.aggregator import LoopbackWorld
    from super_gnn_amd.data_manager import build_loopback_partitions
    from super_gnn_amd.layers import LoopbackSAGE
    rowptr, col, _ = _graph(n=6000, und_edges=40000, seed=4)
    n, Fin, H, C = rowptr.numel() - 1, 64, 128, 8
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n, Fin, generator=gen).cuda()
    y = torch.randint(0, C, (n,), generator=gen).cuda()
    torch.manual_seed(0)
    model = LoopbackSAGE(Fin, H, C, num_layers=3, dropout=0.0).cuda()
    model.reset_parameters()

    def run(P, bits, pre):
        graphs = build_loopback_partitions(rowptr, col, None, P, Fin, num_bits=bits, is_pre_delay=pre)
        world = LoopbackWorld(graphs, bits, pre)
        feats = [x[g.node_range[0]:g.node_range[1]] for g in graphs]
        model.zero_grad()
        out = torch.cat(model(world, feats))
        loss = torch.nn.functional.nll_loss(out, y)
        loss.backward()
        return out.detach(), loss.item(), [p.grad.clone() for p in model.parameters()]

    out1, loss1, g1 = run(1, 32, False)
    for pre in (False, True):
        out4, loss4, g4 = run(4, 32, pre)
        assert torch.allclose(out1, out4, atol=2e-4, rtol=1e-3)
        assert abs(loss1 - loss4) < 1e-4
        for a, b in zip(g1, g4):
            assert torch.allclose(a, b, atol=1e-4, rtol=1e-2)
    # int2 exchange with pre/post aggregation: a few SGD steps reduce the loss
    graphs = build_loopback_partitions(rowptr, col, None, 4, Fin, num_bits=2, is_pre_delay=True)
    world = LoopbackWorld(graphs, 2, True)
    feats = [x[g.node_range[0]:g.node_range[1]] for g in graphs]
    opt = torch.optim.Adam(model.parameters(), lr=5e-3)
    losses = []
    for _ in range(12):
        opt.zero_grad()
        loss = torch.nn.functional.nll_loss(torch.cat(model(world, feats)), y)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < losses[0] - 0.05, losses


def test_world_from_reference_partition_files(tmp_path):
    """Graph -> the reference's per-rank files -> loader -> loop-back world: one int8 aggregation
    equals the global product at the quantization error scale, and the fp32 one within the SpMM bar."""
    from super_gnn_amd.aggregator import LoopbackWorld
    from super_gnn_amd.data_manager import load_loopback_partitions, save_partition_files
    rowptr, col, _ = _graph(n=5000, und_edges=30000, seed=21)
    n, F = rowptr.numel() - 1, 64
    gen = torch.Generator().manual_seed(2)
    feat = torch.randn(n, F, generator=gen)
    label = torch.randint(0, 5, (n,), generator=gen)
    idx = torch.arange(n)
    bounds = torch.tensor([0, 1100, 2600, 3900, n])
    save_partition_files(str(tmp_path), "g", rowptr, col, bounds, feat, label, idx[::3], idx[1::3], idx[2::3])
    rp, c = rowptr.numpy(), col.numpy().astype(np.int64)
    want = np.zeros((n, F), np.float32)
    orc.spmm_accumulate(rp, c, np.ones(c.size, np.float32), feat.numpy(), want)
    for bits, pre in ((32, True), (8, False), (8, True)):
        graphs, data = load_loopback_partitions(str(tmp_path), "g", 4, F, num_bits=bits, is_pre_delay=pre)
        feats = [d["nodes_features"].cuda() for d in data]
        got = torch.cat(LoopbackWorld(graphs, bits, pre).aggregate(feats)).cpu().numpy()
        if bits == 32:
            assert np.all(np.abs(got - want) <= 1e-4 + 1e-5 * np.abs(want))
        else:
            assert np.linalg.norm(got - want) / np.linalg.norm(want) < 0.01


# ------------------------------------------------------------------------------------------------
# the reference's own signatures: Aggregator.apply(graph, feat, layer, num_bits, is_pre_delay, is_training)
# (super_gnn/aggregator.py:15-23) and DistSAGEConvGrad.forward(graph, feat, layer) (layers/sageconv.py:62-89)
# ------------------------------------------------------------------------------------------------
def _global_products(rowptr, col, w, x, G):
    rp, c, v = rowptr.numpy(), col.numpy().astype(np.int64), w.numpy()
    n = rp.shape[0] - 1
    want = np.zeros((n, x.shape[1]), np.float32)
    orc.spmm_accumulate(rp, c, v, x.numpy(), want)
    AT = sp.csr_matrix((v, c, rp), shape=(n, n)).T.tocsr(); AT.sort_indices()
    rpt, ct, vt = AT.indptr.astype(np.int64), AT.indices.astype(np.int64), AT.data.astype(np.float32)
    want_g = np.zeros((n, x.shape[1]), np.float32)
    orc.spmm_accumulate(rpt, ct, vt, G.numpy(), want_g)
    return (rp, c, v, want), (rpt, ct, vt, want_g)


@pytest.mark.parametrize("pre", [False, True])
@pytest.mark.parametrize("P", [1, 4])
def test_reference_signature_aggregator_equals_global_product(pre, P):
    from super_gnn_amd.aggregator import Aggregator, LoopbackWorld
    from super_gnn_amd.data_manager import build_loopback_partitions
    rowptr, col, w = _graph()
    n, F = rowptr.numel() - 1, 64
    graphs = build_loopback_partitions(rowptr, col, w, P, F, num_bits=32, is_pre_delay=pre)
    # world_size == 1: the partition object itself is the graph argument; P > 1: the world of all partitions
    graph = graphs[0] if P == 1 else LoopbackWorld(graphs, 32, pre)
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n, F, generator=gen)
    G = torch.randn(n, F, generator=gen)
    feat = x.cuda().requires_grad_()
    out = Aggregator.apply(graph, feat, 0, 32, pre, True)
    assert out.shape == (n, F)
    out.backward(G.cuda())
    (rp, c, v, want), (rpt, ct, vt, want_g) = _global_products(rowptr, col, w, x, G)
    assert_spmm_close(out.detach().cpu().numpy(), want, orc.spmm_f64(rp, c, v, x.numpy()), abs_sum64(rp, c, v, x.numpy()),
                      np.diff(rp), what="forward")
    assert_spmm_close(feat.grad.cpu().numpy(), want_g, orc.spmm_f64(rpt, ct, vt, G.numpy()), abs_sum64(rpt, ct, vt, G.numpy()),
                      np.diff(rpt), what="backward")
    # the work range the reference caches on the matrix on first use is there (spmm_kernel.py:49-58)
    rs, cs = graphs[0].local_adj_t.get_work_range()
    assert rs.numel() == torch.get_num_threads() + 1 and int(rs[0]) == 0 and int(rs[-1]) == graphs[0].local_adj_t.sparse_size(0)
    assert cs.tolist() == [0, F]


@pytest.mark.parametrize("bits,pre", [(8, False), (2, True), (16, True), (16, False)])
def test_reference_signature_aggregator_equals_loopback_world(bits, pre):
    """Same floats as the list-based world API; eval mode exchanges fp32 rows whatever num_bits says
    (communicator.py:61-62); 16 ships bf16 copies of the boundary rows."""
    from super_gnn_amd.aggregator import Aggregator, LoopbackWorld
    from super_gnn_amd.data_manager import build_loopback_partitions
    rowptr, col, w = _graph(n=8000, und_edges=60000, seed=9)
    n, F, P = rowptr.numel() - 1, 128, 4
    graphs = build_loopback_partitions(rowptr, col, w, P, F, num_bits=bits, is_pre_delay=pre)
    world = LoopbackWorld(graphs, bits, pre)
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(n, F, generator=gen).cuda()
    G = torch.randn(n, F, generator=gen).cuda()
    feat = x.clone().requires_grad_()
    out = Aggregator.apply(world, feat, 1, bits, pre, True)
    out.backward(G)
    if bits != 16:
        feats = [x[g.node_range[0]:g.node_range[1]].clone().requires_grad_() for g in graphs]
        outs = world.aggregate(feats)
        torch.autograd.backward(outs, [G[g.node_range[0]:g.node_range[1]] for g in graphs])
        assert torch.equal(out, torch.cat(outs))
        assert torch.equal(feat.grad, torch.cat([f.grad for f in feats]))
    else:
        # bf16 rows: the exact result with every boundary row rounded to bf16 once, i.e. within 2^-8 relative of
        # the fp32 exchange per contribution; and different from it (the rounding really happened)
        exact = Aggregator.apply(LoopbackWorld(graphs, 32, pre), x, 1, 32, pre, True)
        err = (out.detach() - exact).abs()
        assert float(err.max()) > 0
        xa = x.abs()
        bound = Aggregator.apply(LoopbackWorld(graphs, 32, pre), xa, 1, 32, pre, True) * 2.0 ** -8 + 1e-6
        assert bool((err <= bound).all())
    # evaluation mode: fp32 exchange
    ev = Aggregator.apply(world, x, 1, bits, pre, False)
    ev32 = Aggregator.apply(LoopbackWorld(graphs, 32, pre), x, 1, 32, pre, True)
    assert torch.equal(ev, ev32)
    with pytest.raises(ValueError):
        Aggregator.apply(world, x, 1, bits, not pre, True)
    with pytest.raises(ValueError):
        Aggregator.apply(graphs[0], x[:graphs[0].local_adj_t.sparse_size(0)], 1, bits, pre, True)  # a rank that has peers


def test_reference_signature_sage_layer_and_model():
    from super_gnn_amd.aggregator import LoopbackWorld
    from super_gnn_amd.data_manager import build_loopback_partitions
    from super_gnn_amd.layers import DistSAGE, DistSAGEConvGrad, LoopbackSAGEConv
    rowptr, col, _ = _graph(n=6000, und_edges=40000, seed=3)
    n, F, H, P = rowptr.numel() - 1, 32, 48, 3
    graphs = build_loopback_partitions(rowptr, col, None, P, max(F, H), num_bits=2, is_pre_delay=True)
    world = LoopbackWorld(graphs, 2, True)
    torch.manual_seed(0)
    a = DistSAGEConvGrad(F, H, 2, True).cuda(); a.reset_parameters()
    b = LoopbackSAGEConv(F, H).cuda()
    b.load_state_dict(a.state_dict())
    x = torch.randn(n, F, device="cuda")
    ya = a(world, x, 0)
    yb = torch.cat(b(world, [x[g.node_range[0]:g.node_range[1]] for g in graphs]))
    assert torch.equal(ya, yb)
    # the model trains through the reference's call sequence: model(graph, feats, labels, mask) -> log-probabilities
    model = DistSAGE(F, H, 5, num_layers=3, dropout=0.0, num_bits=2, is_pre_delay=True).cuda()
    model.reset_parameters()
    labels = torch.randint(0, 5, (n,), device="cuda")
    opt = torch.optim.Adam(model.parameters(), lr=0.01)
    losses = []
    for _ in range(8):
        opt.zero_grad()
        loss = torch.nn.functional.nll_loss(model(world, x, labels, None), labels)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < losses[0]
