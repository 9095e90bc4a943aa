"""GCN / GAT layers and the heterogeneous wrapper of the reference's model code
(YiTu_GNN/YiTu_H/test/common/model.py:7-30, 61-106, 137-171), written directly
against the op wrappers instead of the message-passing tracer: same parameters
(names and shapes), same arithmetic.
"""
from typing import Union

import torch
from torch import nn

from . import block, bundle, sparse


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
        h = bundle.linear(x, self.fc.weight, self.fc.bias)
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
            h_src = bundle.linear(x[0], self.linear_v.weight, self.linear_v.bias)
            h_dst = bundle.linear(x[1], self.linear_v.weight, self.linear_v.bias)
        elif isinstance(x, torch.Tensor):
            h_src = h_dst = bundle.linear(x, self.linear_v.weight, self.linear_v.bias)
        else:
            raise TypeError
        if h_dst is h_src:  # one read of h for both projections
            q, k = bundle.linear_pair(h_src, self.linear_q, self.linear_k)
        else:
            q = self.linear_q(h_dst)
            k = self.linear_k(h_src)
        h_src = h_src.view(size=[-1, self.n_heads, self.n_features])
        if self.fused:
            return sparse.fused_gat(blk, q.contiguous(), k.contiguous(), h_src.contiguous(),
                                    head_mean=True)
        else:
            attn = sparse.fused_gsddmm(blk, q.contiguous(), k.contiguous())
            v = sparse.gspmm(blk, attn, h_src.contiguous())
        return torch.mean(v, dim=1)


class GATHeadLayer(nn.Module):
    """GAT layer stated with per-head attention vectors: ``h = linear_v(x)`` viewed as
    [n, H, F] (``in_features=None``: x already is that), logits
    ``LeakyReLU_0.2(<a_dst[h], h_dst> + <a_src[h], h_src>)``, softmax over each
    destination's in-edges, aggregate, mean over heads. The reference's example layer
    (model.py:61-106) makes the two scalars with dense H*F -> H Linears; this is their
    block-diagonal, bias-free case, and runs as one op (``sparse.gat_heads``)."""

    def __init__(self, in_features, out_features: int, n_heads: int, head_mean: bool = True):
        super().__init__()
        self.n_heads, self.n_features, self.head_mean = n_heads, out_features, head_mean
        self.linear_v = None if in_features is None else \
            nn.Linear(in_features, n_heads * out_features)
        self.a_src = nn.Parameter(torch.randn(n_heads, out_features) * 0.1)
        self.a_dst = nn.Parameter(torch.randn(n_heads, out_features) * 0.1)

    def _heads(self, x):
        h = x if self.linear_v is None else \
            bundle.linear(x, self.linear_v.weight, self.linear_v.bias)
        return h.view(size=[-1, self.n_heads, self.n_features])

    def forward(self, blk: block.Block, x):
        if isinstance(x, (list, tuple)):
            assert len(x) == 2
            h_src, h_dst = self._heads(x[0]), self._heads(x[1])
        else:
            h_src, h_dst = self._heads(x), None
        return sparse.gat_heads(blk, h_src, self.a_src, self.a_dst, x_dst=h_dst,
                                head_mean=self.head_mean)


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


class _TypedLinear(torch.autograd.Function):
    """y[off_i : off_i + n_i] = x_i . W_i^T (+ b_i) for every (x_i, W_i, b_i), all
    written into one [sum n_i, out] buffer by the MFMA GEMM: the layout the
    stacked aggregation reads, produced without a concatenation pass."""

    @staticmethod
    def forward(ctx, n_parts, *args):
        from .. import graph_ext
        xs, ws, bs = args[:n_parts], args[n_parts:2 * n_parts], args[2 * n_parts:]
        total = sum(x.size(0) for x in xs)
        y = torch.empty((total, ws[0].size(0)), dtype=torch.float32, device=xs[0].device)
        parts, off = [], 0
        for x in xs:
            parts.append(y[off:off + x.size(0)])
            off += x.size(0)
        if all(w.shape == ws[0].shape for w in ws):
            graph_ext.linear_forward_typed(
                [x.contiguous() for x in xs], [w.contiguous() for w in ws],
                [None if b is None else b.contiguous() for b in bs], out_list=parts)
        else:
            graph_ext.sgemm_typed([x.contiguous() for x in xs], [w.contiguous() for w in ws],
                                  trans_b=True, out_list=parts)
            for part, b in zip(parts, bs):
                if b is not None:
                    part += b
        ctx.n_parts = n_parts
        ctx.has_bias = [b is not None for b in bs]
        ctx.save_for_backward(*xs, *ws)
        return y

    @staticmethod
    def backward(ctx, grad_y):
        from .. import graph_ext
        n = ctx.n_parts
        xs, ws = ctx.saved_tensors[:n], ctx.saved_tensors[n:]
        grad_y = grad_y.contiguous()
        gs, off = [], 0
        for x in xs:
            gs.append(grad_y[off:off + x.size(0)])
            off += x.size(0)
        gx, gw = [None] * n, [None] * n
        want = [i for i in range(n) if ctx.needs_input_grad[1 + i]]
        if want:
            for i, g in zip(want, graph_ext.sgemm_typed([gs[i] for i in want],
                                                        [ws[i].contiguous() for i in want])):
                gx[i] = g
        want = [i for i in range(n) if ctx.needs_input_grad[1 + n + i]]
        if want:
            for i, g in zip(want, graph_ext.sgemm_typed([gs[i] for i in want],
                                                        [xs[i].contiguous() for i in want],
                                                        trans_a=True)):
                gw[i] = g
        gb = [None] * n
        want = [i for i in range(n) if ctx.has_bias[i] and ctx.needs_input_grad[1 + 2 * n + i]]
        if want:
            for i, g in zip(want, graph_ext.column_sum_typed([gs[i] for i in want])):
                gb[i] = g
        return (None, *gx, *gw, *gb)


class StackedHeteroGCN(nn.Module):
    """``HeteroGraphConv`` over ``GCNLayer``s (model.py:137-171 with :7-30) as one
    launch: the transformed features of all source sets sit in one buffer, the
    relations are stacked into one CSR whose edge weights carry
    ``norm[row] / (relations reaching the destination type)``, and a single
    edge-weighted SpMM gives every destination type's output.

    ``ntypes``: {node type: count}; ``relations``: [(src type, edge type, dst
    type)]. ``per_relation=True`` keeps one Linear per edge type like the
    reference's model; ``False`` shares one Linear per source node type (each
    type's features are then transformed once, whatever the number of relations
    leaving it). Parameters: ``fcs[edge type or node type]`` = ``nn.Linear``.
    """

    def __init__(self, ntypes: dict, relations: list, in_features: int, out_features: int,
                 per_relation: bool = True, bias: bool = True):
        super().__init__()
        self.ntypes = dict(ntypes)
        self.relations = [tuple(r) for r in relations]
        self.per_relation = per_relation
        # the feature buffer: one segment per relation (its source type's rows) or per type
        self.segments = ([(ety, sty) for sty, ety, _ in self.relations] if per_relation
                         else [(nty, nty) for nty in self.ntypes])
        self.fcs = nn.ModuleDict({name: nn.Linear(in_features, out_features, bias=bias)
                                  for name, _ in self.segments})
        self.col_offset, off = {}, 0
        for name, nty in self.segments:
            self.col_offset[name] = off
            off += self.ntypes[nty]
        self.n_cols = off
        self.row_offset, off = {}, 0
        for nty in self.ntypes:
            self.row_offset[nty] = off
            off += self.ntypes[nty]
        self.n_rows = off
        self._stacked = None

    def stack(self, hgraph: dict, norms: dict = None):
        """Builds (once per graph) the stacked CSR and its edge weights from
        ``hgraph`` {(src type, edge type, dst type): Block}; ``norms`` as in
        ``HeteroGraphConv`` ({str(key): [n_dst, 1]}), default 1 / in-degree."""
        reach = {}
        for _, _, dty in self.relations:
            reach[dty] = reach.get(dty, 0) + 1
        blocks, rows, cols, scales = [], [], [], []
        for sty, ety, dty in self.relations:
            blk = hgraph[(sty, ety, dty)]
            norm = norms[str((sty, ety, dty))] if norms else right_norm(blk)
            blocks.append(blk)
            rows.append(self.row_offset[dty])
            cols.append(self.col_offset[ety if self.per_relation else sty])
            scales.append(norm.reshape(-1) / reach[dty])
        self._stacked = block.stack_blocks(blocks, rows, cols, self.n_rows, self.n_cols, scales)
        return self._stacked

    def forward(self, xs: dict, stacked=None):
        blk, values = stacked if stacked is not None else self._stacked
        parts = [xs[nty] for _, nty in self.segments]
        fcs = [self.fcs[name] for name, _ in self.segments]
        h = _TypedLinear.apply(len(parts), *parts, *[fc.weight for fc in fcs],
                               *[fc.bias for fc in fcs])
        out = sparse.gspmm(blk, values, h.unsqueeze(1)).squeeze(1)
        reached = {dty for _, _, dty in self.relations}
        # one split (its backward is one concatenation) rather than a slice per type (each
        # slice's backward would be a zero-filled buffer of the full height)
        pieces = out.split(list(self.ntypes.values()))
        return {nty: piece for nty, piece in zip(self.ntypes, pieces) if nty in reached}
