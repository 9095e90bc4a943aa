"""The reference's example models written against the message-passing front end
(YiTu_GNN/YiTu_H/test/common/model.py): same parameter names and arithmetic, so a
state dict moves between the two. They run three ways: eagerly on real tensors
(``mp.Graph`` computes each message function directly), traced and executed as
captured, or traced, lowered (and stitched) onto the HIP ops.
"""
from typing import Union

import torch
from torch import nn

from . import mp


class GCNLayer(nn.Module):
    """norm * sum_{u -> v} fc(x)[u] (model.py:7-30)."""

    def __init__(self, in_features: int, out_features: int):
        super().__init__()
        self.fc = nn.Linear(in_features, out_features)

    def forward(self, graph: mp.Graph, norm: torch.Tensor, x: Union[torch.Tensor, list]):
        if isinstance(x, (list, tuple)):
            assert len(x) == 2
            x = x[0]
        h = self.fc(x)
        graph.src_node["u"] = h.view(size=[-1, 1, h.size(-1)])
        graph.message_func(mp.Fn.copy_u("u", "m"))
        graph.reduce_func(mp.Fn.aggregate_sum("m", "v"))
        return torch.multiply(norm, torch.squeeze(graph.dst_node["v"], dim=1))


class GATLayer(nn.Module):
    """Additive attention with dense H*F -> H projections for query and key, mean
    over heads (model.py:61-106)."""

    def __init__(self, in_features: int, out_features: int, n_heads: int):
        super().__init__()
        self.n_heads = n_heads
        self.n_features = out_features
        self.linear_q = nn.Linear(n_heads * out_features, n_heads)
        self.linear_k = nn.Linear(n_heads * out_features, n_heads)
        self.linear_v = nn.Linear(in_features, n_heads * out_features)
        self.leaky_relu = nn.LeakyReLU(negative_slope=0.2)

    def forward(self, graph: mp.Graph, x):
        if isinstance(x, (list, tuple)):
            assert len(x) == 2
            h_src, h_dst = self.linear_v(x[0]), self.linear_v(x[1])
        elif isinstance(x, torch.Tensor):
            h_src = h_dst = self.linear_v(x)
        else:
            raise TypeError(type(x))
        # the reference files the query under src_node and the key under dst_node
        # (model.py:91-92); names are resolved across all stores, so it does not matter
        graph.src_node["q"] = self.linear_q(h_dst)
        graph.dst_node["k"] = self.linear_k(h_src)
        graph.src_node["u"] = h_src.view(size=[-1, self.n_heads, self.n_features])
        graph.message_func(mp.Fn.u_add_v("k", "q", "e"))
        graph.edge["coeff"] = self.leaky_relu(graph.edge["e"])
        graph.message_func(mp.Fn.edge_softmax("coeff", "attn"))
        graph.message_func(mp.Fn.u_mul_e("u", "attn", "m"))
        graph.reduce_func(mp.Fn.aggregate_sum("m", "v"))
        return torch.mean(graph.dst_node["v"], dim=1)


class GCNModel(nn.Module):
    """model.py:33-58"""

    def __init__(self, in_features: int, gnn_features: int, out_features: int):
        super().__init__()
        self.i2h = GCNLayer(in_features, gnn_features)
        self.h2o = GCNLayer(gnn_features, out_features)
        self.activation = nn.Sequential(nn.Dropout(0.5), nn.ReLU())

    def forward(self, graph: mp.Graph, x: torch.Tensor, norm: torch.Tensor):
        h = self.activation(self.i2h(graph, norm, x))
        return self.h2o(graph, norm, h)


class GATModel(nn.Module):
    """model.py:109-134"""

    def __init__(self, in_features: int, gnn_features: int, out_features: int, n_heads: int = 8):
        super().__init__()
        self.i2h = GATLayer(in_features, gnn_features, n_heads=n_heads)
        self.h2o = GATLayer(gnn_features, out_features, n_heads=n_heads)
        self.activation = nn.Sequential(nn.Dropout(0.5), nn.ELU())

    def forward(self, graph: mp.Graph, x: torch.Tensor):
        return self.h2o(graph, self.activation(self.i2h(graph, x)))


class HeteroGraphConv(nn.Module):
    """One conv per edge type, averaged over the relations that reach each
    destination type (model.py:137-171)."""

    def __init__(self, convs: dict):
        super().__init__()
        self.convs = nn.ModuleDict(convs)

    def forward(self, hgraph: mp.HeteroGraph, xs: dict, norms: dict = None):
        counts, outputs = {}, {}
        for (sty, ety, dty), graph in hgraph:
            pair = (xs[sty], xs[dty])
            if norms:
                res = self.convs[ety](graph, norms[str((sty, ety, dty))], pair)
            else:
                res = self.convs[ety](graph, pair)
            counts[dty] = counts.get(dty, 0) + 1
            outputs[dty] = res if dty not in outputs else outputs[dty] + res
        return {dty: res / counts[dty] for dty, res in outputs.items()}


class REmbedding(nn.Module):
    """A learned embedding table per node type (model.py:174-195)."""

    def __init__(self, hgraph: mp.HeteroGraph, embedding_dim: int):
        super().__init__()
        self.embeds = nn.ModuleDict({nty: nn.Embedding(num, embedding_dim)
                                     for nty, num in hgraph.nty2num.items()})

    def forward(self, hgraph: mp.HeteroGraph, xs: dict):
        return {nty: self.embeds[nty](xs[nty]) for nty in hgraph.nty2num}


class RGCNModel(nn.Module):
    """model.py:198-236"""

    def __init__(self, hgraph: mp.HeteroGraph, in_features: int, gnn_features: int,
                 out_features: int):
        super().__init__()
        self.em = REmbedding(hgraph, in_features)
        self.i2h = HeteroGraphConv({ety: GCNLayer(in_features, gnn_features)
                                    for ety in hgraph.etypes})
        self.h2o = HeteroGraphConv({ety: GCNLayer(gnn_features, out_features)
                                    for ety in hgraph.etypes})
        self.activation = nn.Sequential(nn.Dropout(0.5), nn.ReLU())

    def forward(self, hgraph: mp.HeteroGraph, norms: dict, xs: dict):
        hs = self.i2h(hgraph, self.em(hgraph, xs), norms)
        hs = {k: self.activation(h) for k, h in hs.items()}
        return self.h2o(hgraph, hs, norms)


class RGATModel(nn.Module):
    """model.py:239-285"""

    def __init__(self, hgraph: mp.HeteroGraph, in_features: int, gnn_features: int,
                 out_features: int, n_heads: int = 8):
        super().__init__()
        self.em = REmbedding(hgraph, in_features)
        self.i2h = HeteroGraphConv({ety: GATLayer(in_features, gnn_features, n_heads=n_heads)
                                    for ety in hgraph.etypes})
        self.h2o = HeteroGraphConv({ety: GATLayer(gnn_features, out_features, n_heads=n_heads)
                                    for ety in hgraph.etypes})
        self.activation = nn.Sequential(nn.Dropout(0.5), nn.ELU())

    def forward(self, hgraph: mp.HeteroGraph, xs: dict):
        hs = self.i2h(hgraph, self.em(hgraph, xs))
        hs = {k: self.activation(h) for k, h in hs.items()}
        return self.h2o(hgraph, hs)
