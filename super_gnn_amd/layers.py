"""GraphSAGE layer and model over the loop-back partitions: the arithmetic of the reference's
``DistSAGEConvGrad.forward`` (super_gnn/layers/sageconv.py:62-89: aggregate, divide by the in-degree,
``lin_neigh(agg) + lin_self(x) + bias``) and of ``DistSAGE.forward`` (examples/graphsage/sage.py:176-211:
conv, dropout, norm, relu per hidden layer, log_softmax at the end), with every partition of the
graph processed in this one process and the weights shared between them (what DistributedDataParallel
replication amounts to on one GPU).  The dense products are plain torch (rocBLAS) GEMMs."""
import math
from typing import List, Sequence

import torch
import torch.nn.functional as F
from torch import Tensor
from torch.nn import LayerNorm, Linear, Parameter

from .aggregator import Aggregator, LoopbackWorld


def _column_sum(g: Tensor) -> Tensor:
    n, c = g.shape
    k = 4 // math.gcd(c, 4)
    if k == 1 or n < k or not g.is_contiguous():
        return g.sum(0)
    m = n // k * k
    s = g[:m].view(m // k, k * c).sum(0).view(k, c).sum(0)
    return s + g[m:].sum(0) if m < n else s


_SPLIT_K = 64


def _weight_grad(g: Tensor, a: Tensor) -> Tensor:
    """g^T @ a for tall operands ([rows, out] and [rows, in], rows >> out, in).  The product has only
    out x in outputs, too few tiles to fill 256 CUs, so the row axis is cut into _SPLIT_K slabs that run as one
    batched GEMM and are then added (measured at 306 k rows: 0.67 -> 0.17 ms for 256 x 128, 0.71 -> 0.32 ms for
    256 x 256, 0.78 -> 0.11 ms for 47 x 256)."""
    n = g.shape[0]
    if n < _SPLIT_K * 1024 or not (g.is_contiguous() and a.is_contiguous()):
        return g.t() @ a
    m = n // _SPLIT_K * _SPLIT_K
    w = torch.bmm(g[:m].view(_SPLIT_K, m // _SPLIT_K, -1).transpose(1, 2), a[:m].view(_SPLIT_K, m // _SPLIT_K, -1)).sum(0)
    if m < n:
        w.addmm_(g[m:].t(), a[m:])
    return w


class _SageCombine(torch.autograd.Function):
    """``(agg / deg) @ W_neigh^T + x @ W_self^T + bias`` (sageconv.py:83-89) as two GEMMs that accumulate into one
    output, instead of two products and two elementwise additions.  In the backward pass the bias gradient is
    summed through a [rows / 4, 4 * width] view when the width is not a multiple of 4: torch's column sum of
    a tall [rows, 47] matrix takes 2.4 ms per partition on MI355X (scalar loads), the same bytes viewed
    188 wide take the vectorized path."""

    @staticmethod
    def forward(ctx, agg, x, deg, w_neigh, w_self, bias):
        mean = agg / deg if deg is not None else agg
        out = torch.addmm(bias, x, w_self.t()) if bias is not None else x @ w_self.t()
        out.addmm_(mean, w_neigh.t())
        ctx.save_for_backward(mean, x, deg, w_neigh, w_self)
        ctx.has_bias = bias is not None
        return out

    @staticmethod
    def backward(ctx, g):
        mean, x, deg, w_neigh, w_self = ctx.saved_tensors
        g = g.contiguous()
        need = ctx.needs_input_grad
        g_agg = g_x = g_wn = g_ws = g_b = None
        if need[0]:
            g_agg = g @ w_neigh
            if deg is not None:
                g_agg.div_(deg)
        if need[1]:
            g_x = g @ w_self
        if need[3]:
            g_wn = _weight_grad(g, mean)
        if need[4]:
            g_ws = _weight_grad(g, x)
        if ctx.has_bias and need[5]:
            g_b = _column_sum(g)
        return g_agg, g_x, None, g_wn, g_ws, g_b


class LoopbackSAGEConv(torch.nn.Module):
    def __init__(self, in_channels: int, out_channels: int, normalize: bool = True, bias: bool = True):
        super().__init__()
        self.in_channels, self.out_channels, self.normalize = in_channels, out_channels, normalize
        self.lin_neigh = Linear(in_channels, out_channels, bias=False)
        self.lin_self = Linear(in_channels, out_channels, bias=False)
        if bias:
            self.bias = Parameter(torch.zeros(out_channels))
        else:
            self.register_parameter("bias", None)

    def reset_parameters(self):
        gain = torch.nn.init.calculate_gain("relu")
        torch.nn.init.xavier_uniform_(self.lin_neigh.weight, gain=gain)
        torch.nn.init.xavier_uniform_(self.lin_self.weight, gain=gain)

    def forward(self, world: LoopbackWorld, feats: Sequence[Tensor]) -> List[Tensor]:
        aggregated = world.aggregate(feats)
        outs = []
        for g, agg, x in zip(world.graphs, aggregated, feats):
            outs.append(_SageCombine.apply(agg, x, g.in_degrees if self.normalize else None,
                                           self.lin_neigh.weight, self.lin_self.weight, self.bias))
        return outs


class LoopbackSAGE(torch.nn.Module):
    def __init__(self, in_channels, hidden_channels, out_channels, num_layers=3, dropout=0.5, norm_type="LayerNorm"):
        super().__init__()
        dims = [in_channels] + [hidden_channels] * (num_layers - 1) + [out_channels]
        self.convs = torch.nn.ModuleList(LoopbackSAGEConv(a, b) for a, b in zip(dims[:-1], dims[1:]))
        self.norms = torch.nn.ModuleList(LayerNorm(hidden_channels) for _ in range(num_layers - 1)) \
            if norm_type == "LayerNorm" else None
        self.dropout = dropout

    def reset_parameters(self):
        for conv in self.convs:
            conv.reset_parameters()
        if self.norms is not None:
            for norm in self.norms:
                norm.reset_parameters()

    def forward(self, world: LoopbackWorld, feats: Sequence[Tensor]) -> List[Tensor]:
        for i, conv in enumerate(self.convs[:-1]):
            feats = conv(world, feats)
            feats = [F.dropout(x, p=self.dropout, training=self.training) for x in feats]
            if self.norms is not None:
                feats = [self.norms[i](x) for x in feats]
            feats = [F.relu(x) for x in feats]
        feats = self.convs[-1](world, feats)
        return [F.log_softmax(x, dim=1) for x in feats]


class DistSAGEConvGrad(torch.nn.Module):
    """The reference's layer with the reference's constructor and call signatures
    (super_gnn/layers/sageconv.py:15-89): ``conv(graph, local_nodes_feat, layer)`` aggregates through
    ``Aggregator.apply(graph, feat, layer, num_bits, is_pre_delay, self.training)``, divides by
    ``graph.in_degrees`` and returns ``lin_neigh(agg) + lin_self(feat) + bias``.  ``graph`` is whatever
    ``Aggregator`` accepts: a partition that is the whole graph, or a LoopbackWorld of P partitions with the
    node features of all of them stacked in partition order."""

    def __init__(self, in_channels: int, out_channels: int, num_bits: int, is_pre_delay: bool,
                 add_self_loops: bool = False, normalize: bool = True, bias: bool = True, **kwargs):
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.add_self_loops, self.normalize = add_self_loops, normalize
        self.num_bits, self.is_pre_delay = num_bits, is_pre_delay
        self.lin_neigh = Linear(in_channels, out_channels, bias=False)
        self.lin_self = Linear(in_channels, out_channels, bias=False)
        if bias:
            self.bias = Parameter(torch.zeros(out_channels))
        else:
            self.register_parameter("bias", None)

    def reset_parameters(self):
        gain = torch.nn.init.calculate_gain("relu")
        torch.nn.init.xavier_uniform_(self.lin_neigh.weight, gain=gain)
        torch.nn.init.xavier_uniform_(self.lin_self.weight, gain=gain)

    def propagate(self, graph, local_nodes_feat, layer):
        return Aggregator.apply(graph, local_nodes_feat, layer, self.num_bits, self.is_pre_delay, self.training)

    def forward(self, graph, local_nodes_feat, layer) -> Tensor:
        agg = self.propagate(graph, local_nodes_feat, layer)
        deg = graph.in_degrees.reshape(-1, 1) if self.normalize else None
        return _SageCombine.apply(agg, local_nodes_feat, deg, self.lin_neigh.weight, self.lin_self.weight, self.bias)


class DistSAGE(torch.nn.Module):
    """The model of the reference's training script with its constructor and call signatures
    (examples/graphsage/sage.py:127-211; LayerNorm or no norm, no label augmentation)."""

    def __init__(self, in_channels, hidden_channels, out_channels, num_layers=3, dropout=0.5, num_bits=32,
                 is_pre_delay=False, norm_type="LayerNorm", is_label_augment=False):
        super().__init__()
        if is_label_augment:
            raise NotImplementedError("label augmentation (MaskLabel) is outside the aggregation hot path")
        if norm_type not in (None, "LayerNorm"):
            raise NotImplementedError("only LayerNorm (the reference's default) or no normalisation")
        dims = [in_channels] + [hidden_channels] * (num_layers - 1) + [out_channels]
        self.convs = torch.nn.ModuleList(DistSAGEConvGrad(a, b, num_bits, is_pre_delay) for a, b in zip(dims[:-1], dims[1:]))
        self.norms = torch.nn.ModuleList(LayerNorm(hidden_channels) for _ in range(num_layers - 1)) if norm_type else None
        self.dropout, self.norm_type = dropout, norm_type

    def reset_parameters(self):
        for conv in self.convs:
            conv.reset_parameters()
        if self.norms is not None:
            for norm in self.norms:
                norm.reset_parameters()

    def forward(self, graph, nodes_feats, labels=None, label_mask=None):
        for i, conv in enumerate(self.convs[:-1]):
            nodes_feats = conv(graph, nodes_feats, i)
            nodes_feats = F.dropout(nodes_feats, p=self.dropout, training=self.training)
            if self.norms is not None:
                nodes_feats = self.norms[i](nodes_feats)
            nodes_feats = F.relu(nodes_feats)
        nodes_feats = self.convs[-1](graph, nodes_feats, len(self.convs) - 1)
        return F.log_softmax(nodes_feats, dim=1)
