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


def sum_neighbours(graph: mp.Graph, x: torch.Tensor, weights: str = None) -> torch.Tensor:
    """Message passing recipe shared by the layers: every destination sums the
    rows ``x [n_src, H, F]`` of its in-neighbours, scaled per edge and head by the
    edge tensor named ``weights`` when given. Returns [n_dst, H, F]."""
    graph.src_node["u"] = x
    if weights is None:
        graph.message_func(mp.Fn.copy_u("u", "m"))
    else:
        graph.message_func(mp.Fn.u_mul_e("u", weights, "m"))
    graph.reduce_func(mp.Fn.aggregate_sum("m", "v"))
    return graph.dst_node["v"]


def _source_side(x):
    """Layers of a heterogeneous model receive (source features, destination features)."""
    if isinstance(x, (list, tuple)):
        assert len(x) == 2
        return x[0], x[1]
    if isinstance(x, torch.Tensor):
        return x, x
    raise TypeError(type(x))


class GCNLayer(nn.Module):
    """norm * sum_{u -> v} fc(x)[u] (model.py:7-30). Parameters: ``fc``."""

    def __init__(self, in_features: int, out_features: int):
        super().__init__()
        self.fc = nn.Linear(in_features, out_features)

    def forward(self, graph: mp.Graph, norm: torch.Tensor, x: Union[torch.Tensor, list]):
        x_src, _ = _source_side(x)
        h = self.fc(x_src)
        total = sum_neighbours(graph, h.view(size=[-1, 1, h.size(-1)]))
        return torch.multiply(norm, torch.squeeze(total, dim=1))


class GATLayer(nn.Module):
    """Additive attention, mean over heads (model.py:61-106). Parameters:
    ``linear_v`` (in -> H*F), ``linear_q`` / ``linear_k`` (dense H*F -> H, applied
    to the transformed destination / source features), ``leaky_relu`` (0.2)."""

    def __init__(self, in_features: int, out_features: int, n_heads: int):
        super().__init__()
        self.n_heads, self.n_features = n_heads, out_features
        width = n_heads * out_features
        self.linear_q = nn.Linear(width, n_heads)
        self.linear_k = nn.Linear(width, n_heads)
        self.linear_v = nn.Linear(in_features, width)
        self.leaky_relu = nn.LeakyReLU(negative_slope=0.2)

    def forward(self, graph: mp.Graph, x):
        x_src, x_dst = _source_side(x)
        h_src = self.linear_v(x_src)
        h_dst = h_src if x_dst is x_src else self.linear_v(x_dst)
        # names are resolved across the node stores, so where the reference files the
        # query and the key (src_node / dst_node, model.py:91-92) is immaterial
        graph.dst_node["q"] = self.linear_q(h_dst)
        graph.src_node["k"] = self.linear_k(h_src)
        graph.message_func(mp.Fn.u_add_v("k", "q", "e"))
        graph.edge["coeff"] = self.leaky_relu(graph.edge["e"])
        graph.message_func(mp.Fn.edge_softmax("coeff", "attn"))
        heads = h_src.view(size=[-1, self.n_heads, self.n_features])
        return torch.mean(sum_neighbours(graph, heads, weights="attn"), dim=1)


def _between_layers(nonlinearity: nn.Module) -> nn.Sequential:
    # the reference's models put Dropout(0.5) and the nonlinearity between their two layers
    return nn.Sequential(nn.Dropout(0.5), nonlinearity)


class GCNModel(nn.Module):
    """Two GCN layers on one graph (model.py:33-58): ``i2h``, ``h2o``, ``activation``."""

    def __init__(self, in_features: int, gnn_features: int, out_features: int):
        super().__init__()
        self.i2h = GCNLayer(in_features, gnn_features)
        self.h2o = GCNLayer(gnn_features, out_features)
        self.activation = _between_layers(nn.ReLU())

    def forward(self, graph: mp.Graph, x: torch.Tensor, norm: torch.Tensor):
        hidden = self.activation(self.i2h(graph, norm, x))
        return self.h2o(graph, norm, hidden)


class GATModel(nn.Module):
    """Two GAT layers on one graph (model.py:109-134)."""

    def __init__(self, in_features: int, gnn_features: int, out_features: int, n_heads: int = 8):
        super().__init__()
        self.i2h = GATLayer(in_features, gnn_features, n_heads=n_heads)
        self.h2o = GATLayer(gnn_features, out_features, n_heads=n_heads)
        self.activation = _between_layers(nn.ELU())

    def forward(self, graph: mp.Graph, x: torch.Tensor):
        return self.h2o(graph, self.activation(self.i2h(graph, x)))


class HeteroGraphConv(nn.Module):
    """One layer per edge type (``convs[edge type]``); a destination type's result
    is the mean over the relations that reach it (model.py:137-171)."""

    def __init__(self, convs: dict):
        super().__init__()
        self.convs = nn.ModuleDict(convs)

    def forward(self, hgraph: mp.HeteroGraph, xs: dict, norms: dict = None):
        per_type = {}
        for rel, graph in hgraph:
            sty, ety, dty = rel
            args = (graph, norms[str(rel)]) if norms else (graph,)
            per_type.setdefault(dty, []).append(self.convs[ety](*args, (xs[sty], xs[dty])))
        means = {}
        for dty, terms in per_type.items():
            total = terms[0]
            for t in terms[1:]:
                total = total + t
            means[dty] = total / len(terms)
        return means


class REmbedding(nn.Module):
    """A learned table per node type, indexed by node id (model.py:174-195)."""

    def __init__(self, hgraph: mp.HeteroGraph, embedding_dim: int):
        super().__init__()
        self.embeds = nn.ModuleDict()
        for nty, count in hgraph.nty2num.items():
            self.embeds[nty] = nn.Embedding(count, embedding_dim)

    def forward(self, hgraph: mp.HeteroGraph, xs: dict):
        return {nty: table(xs[nty]) for nty, table in self.embeds.items()}


class _TwoHeteroLayers(nn.Module):
    """Embedding, a heterogeneous layer, Dropout + nonlinearity, a second layer."""

    def __init__(self, hgraph, widths, make_layer, nonlinearity):
        super().__init__()
        d_in, d_hidden, d_out = widths
        self.em = REmbedding(hgraph, d_in)
        self.i2h = HeteroGraphConv({ety: make_layer(d_in, d_hidden) for ety in hgraph.etypes})
        self.h2o = HeteroGraphConv({ety: make_layer(d_hidden, d_out) for ety in hgraph.etypes})
        self.activation = _between_layers(nonlinearity)

    def _run(self, hgraph, xs, norms):
        hidden = self.i2h(hgraph, self.em(hgraph, xs), norms)
        hidden = {nty: self.activation(h) for nty, h in hidden.items()}
        return self.h2o(hgraph, hidden, norms)


class RGCNModel(_TwoHeteroLayers):
    """model.py:198-236"""

    def __init__(self, hgraph: mp.HeteroGraph, in_features: int, gnn_features: int,
                 out_features: int):
        super().__init__(hgraph, (in_features, gnn_features, out_features), GCNLayer, nn.ReLU())

    def forward(self, hgraph: mp.HeteroGraph, norms: dict, xs: dict):
        return self._run(hgraph, xs, norms)


class RGATModel(_TwoHeteroLayers):
    """model.py:239-285"""

    def __init__(self, hgraph: mp.HeteroGraph, in_features: int, gnn_features: int,
                 out_features: int, n_heads: int = 8):
        super().__init__(hgraph, (in_features, gnn_features, out_features),
                         lambda i, o: GATLayer(i, o, n_heads=n_heads), nn.ELU())

    def forward(self, hgraph: mp.HeteroGraph, xs: dict):
        return self._run(hgraph, xs, None)
