"""GraphSAGE layer and model over the loop-back partitions: the arithmetic of the reference's
``DistSAGEConvGrad.forward`` (super_gnn/layers/sageconv.py:62-89: aggregate, divide by the in-degree,
``lin_neigh(agg) + lin_self(x) + bias``) and of ``DistSAGE.forward`` (examples/graphsage/sage.py:176-211:
conv, dropout, norm, relu per hidden layer, log_softmax at the end), with every partition of the
graph processed in this one process and the weights shared between them (what DistributedDataParallel
replication amounts to on one GPU).  The dense products are plain torch (rocBLAS) GEMMs."""
from typing import List, Sequence

import torch
import torch.nn.functional as F
from torch import Tensor
from torch.nn import LayerNorm, Linear, Parameter

from .aggregator import LoopbackWorld


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
            if self.normalize:
                agg = agg / g.in_degrees
            out = self.lin_neigh(agg) + self.lin_self(x)
            if self.bias is not None:
                out = out + self.bias
            outs.append(out)
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
