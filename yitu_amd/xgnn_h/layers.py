"""GCN / GAT layers and the heterogeneous wrapper of the reference's model code
(YiTu_GNN/YiTu_H/test/common/model.py:7-30, 61-106, 137-171), written directly
against the op wrappers instead of the message-passing tracer: same parameters
(names and shapes), same arithmetic.
"""
from typing import Union

import torch
from torch import nn

from . import block, sparse


def right_norm(blk: block.Block):
    """1 / in-degree as [n_dst, 1] (xgnn_h/mp.py:165-167); 0 for rows without
    edges, where the reference produces inf (and then 0 * inf = NaN)."""
    indptr = blk.adj_sparse[0]
    deg = (indptr[1:] - indptr[:-1]).to(torch.float32)
    return torch.where(deg > 0, 1.0 / deg.clamp(min=1.0), torch.zeros_like(deg)).unsqueeze(-1)


class GCNLayer(nn.Module):
    """fc(x) -> copy_u / aggregate_sum -> multiply by norm (model.py:7-30)."""

    def __init__(self, in_features: int, out_features: int):
        super().__init__()
        self.fc = nn.Linear(in_features, out_features)

    def forward(self, blk: block.Block, norm: torch.Tensor, x: Union[torch.Tensor, list]):
        if isinstance(x, (list, tuple)):
            assert len(x) == 2
            x = x[0]
        h = self.fc(x)
        h = h.view(size=[-1, 1, h.size(-1)])
        h = torch.squeeze(sparse.gspmm(blk, None, h), dim=1)
        return torch.multiply(norm, h)


class GATLayer(nn.Module):
    """h = linear_v(x); q = linear_q(h_dst), k = linear_k(h_src) (full H*F -> H
    Linears with bias); u_add_v -> LeakyReLU(0.2) -> edge_softmax -> u_mul_e ->
    aggregate_sum; mean over heads (model.py:61-106). ``fused=True`` runs the
    attention as the single fused op, ``False`` as the reference's two ops."""

    def __init__(self, in_features: int, out_features: int, n_heads: int, fused: bool = True):
        super().__init__()
        self.n_heads = n_heads
        self.n_features = out_features
        self.fused = fused
        self.linear_q = nn.Linear(n_heads * out_features, n_heads)
        self.linear_k = nn.Linear(n_heads * out_features, n_heads)
        self.linear_v = nn.Linear(in_features, n_heads * out_features)
        self.leaky_relu = nn.LeakyReLU(negative_slope=0.2)

    def forward(self, blk: block.Block, x):
        if isinstance(x, (list, tuple)):
            assert len(x) == 2
            h_src = self.linear_v(x[0])
            h_dst = self.linear_v(x[1])
        elif isinstance(x, torch.Tensor):
            h_src = h_dst = self.linear_v(x)
        else:
            raise TypeError
        q = self.linear_q(h_dst)
        k = self.linear_k(h_src)
        h_src = h_src.view(size=[-1, self.n_heads, self.n_features])
        if self.fused:
            v = sparse.fused_gat(blk, q.contiguous(), k.contiguous(), h_src.contiguous())
        else:
            attn = sparse.fused_gsddmm(blk, q.contiguous(), k.contiguous())
            v = sparse.gspmm(blk, attn, h_src.contiguous())
        return torch.mean(v, dim=1)


class HeteroGraphConv(nn.Module):
    """One conv per edge type; results summed per destination type and divided by
    the number of relations that reach it (model.py:137-171). ``hgraph`` maps
    (src type, edge type, dst type) -> Block."""

    def __init__(self, convs: dict):
        super().__init__()
        self.convs = nn.ModuleDict(convs)

    def forward(self, hgraph: dict, xs: dict, norms: dict = None):
        counts, outputs = {}, {}
        for (sty, ety, dty), blk in hgraph.items():
            if norms:
                res = self.convs[ety](blk, norms[str((sty, ety, dty))], (xs[sty], xs[dty]))
            else:
                res = self.convs[ety](blk, (xs[sty], xs[dty]))
            counts[dty] = counts.get(dty, 0) + 1
            outputs[dty] = res if dty not in outputs else outputs[dty] + res
        for dty, res in outputs.items():
            outputs[dty] = res / counts[dty]
        return outputs
