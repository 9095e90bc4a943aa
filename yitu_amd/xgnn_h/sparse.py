"""Differentiable sparse ops over a ``Block`` (the role of xgnn_h/sparse.py): the
same Function classes and wrappers, each a thin autograd shell around one pair of
``graph_ext`` calls. The sparse structure never takes a gradient; a gradient that
the caller does not need is not computed."""
import torch
from torch import autograd
from torch.autograd.function import once_differentiable

from .. import graph_ext
from . import block


def _structure_is_constant(ctx):
    # the [indptr, indices] pair is passed through autograd as a plain list
    assert ctx.needs_input_grad[0] is False


class GSPMMFunction(autograd.Function):
    """out[r,h,:] = sum_e values[e,h] x[col_e,h,:] (sparse.py:7-35)."""

    @staticmethod
    def forward(ctx, adj_sparse, adj_values, x):
        ctx.adj_sparse = adj_sparse
        ctx.save_for_backward(adj_values, x)
        return graph_ext.spmm_forward(adj_values, adj_sparse[0], adj_sparse[1], x)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        _structure_is_constant(ctx)
        assert len(ctx.needs_input_grad) == 3
        values, x = ctx.saved_tensors
        grad_values, grad_x = graph_ext.spmm_backward(
            values, ctx.adj_sparse[0], ctx.adj_sparse[1], x, grad_out.contiguous(),
            need_grad_a=ctx.needs_input_grad[1], need_grad_x=ctx.needs_input_grad[2])
        return None, grad_values, grad_x


def gspmm(block: block.Block, edge: torch.Tensor, x: torch.Tensor):
    """Edge-weighted aggregation of ``x [n_src, H, F]``; ``edge=None`` means unit
    weights (sparse.py:38-51)."""
    assert x.dim() == 3
    if edge is None:
        n_edges = block.adj_sparse[1].size(0)
        edge = torch.ones(size=[n_edges, x.size(1)], device=x.device)
    return GSPMMFunction.apply(block.adj_sparse, edge, x)


class GSDDMMFunction(autograd.Function):
    """attn = softmax_row(LeakyReLU(query[bid,row] + key[col])) (sparse.py:54-81)."""

    @staticmethod
    def forward(ctx, adj_sparse, query, key):
        ctx.adj_sparse = adj_sparse
        attn = graph_ext.sddmm_forward(adj_sparse[0], adj_sparse[1], query, key)
        ctx.save_for_backward(query, key, attn)
        return attn

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_attn):
        _structure_is_constant(ctx)
        # like the reference, both projections are expected to train
        assert ctx.needs_input_grad[1:] == (True, True)
        query, key, attn = ctx.saved_tensors
        grad_query, grad_key = graph_ext.sddmm_backward(
            ctx.adj_sparse[0], ctx.adj_sparse[1], query, key, attn, grad_attn.contiguous())
        return None, grad_query, grad_key


def fused_gsddmm(block: block.Block, query: torch.Tensor, key: torch.Tensor):
    """``query`` [n_dst, H] or, for a stitched block, [n_blocks, n_dst, H]
    (sparse.py:84-91)."""
    query = query if query.dim() == 3 else query.unsqueeze(0)
    return GSDDMMFunction.apply(block.adj_sparse, query, key)


class HFUSEDFunction(autograd.Function):
    """An SpMM on one block and an SDDMM on another, issued together
    (sparse.py:94-110), with the backward the reference leaves unimplemented."""

    @staticmethod
    def forward(ctx, spmm_sparse, spmm_values, spmm_x, sddmm_sparse, sddmm_query, sddmm_key):
        ctx.structures = (spmm_sparse, sddmm_sparse)
        out, attn = graph_ext.hfused_forward(spmm_values, *spmm_sparse, spmm_x, *sddmm_sparse,
                                             sddmm_query, sddmm_key)
        ctx.save_for_backward(spmm_values, spmm_x, sddmm_query, sddmm_key, attn)
        return out, attn

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_spmm, grad_attn):
        (a_ptr, a_idx), (b_ptr, b_idx) = ctx.structures
        values, x, query, key, attn = ctx.saved_tensors
        grad_values, grad_x, grad_query, grad_key = graph_ext.hfused_backward(
            values, a_ptr, a_idx, x, grad_spmm.contiguous(),
            b_ptr, b_idx, query, key, attn, grad_attn.contiguous())
        return None, grad_values, grad_x, None, grad_query, grad_key


def hfused_spddmm(spmm_block: block.Block, spmm_values, spmm_x, sddmm_block: block.Block,
                  sddmm_query, sddmm_key):
    """sparse.py:113-120"""
    if sddmm_query.dim() == 2:
        sddmm_query = sddmm_query.unsqueeze(0)
    return HFUSEDFunction.apply(spmm_block.adj_sparse, spmm_values, spmm_x,
                                sddmm_block.adj_sparse, sddmm_query, sddmm_key)


class FusedGATFunction(autograd.Function):
    """The vertical fusion the reference's optimizer stops short of:
    ``gspmm(blk, fused_gsddmm(blk, q, k), x)`` as one op, forward and backward, and
    optionally the mean over heads that the layer applies next (model.py:106): its
    gradient is then one F-float row per destination, which the backward gathers
    as it is instead of H * F floats per edge."""

    @staticmethod
    def forward(ctx, adj_sparse, query, key, x, head_mean):
        indptr, indices = adj_sparse
        # one-pass shapes: keep each row's softmax statistics instead of the probabilities
        ctx.stats_only = graph_ext.gat_one_pass_shape(x.size(1), x.size(2)) and \
            indices.numel() > 0
        out, attn, *stats = graph_ext.gat_forward(indptr, indices, query, key, x,
                                                  stats_only=ctx.stats_only)
        ctx.adj_sparse = adj_sparse
        ctx.head_mean = head_mean
        ctx.save_for_backward(query, key, x, stats[0] if ctx.stats_only else attn, out)
        return out.mean(dim=1) if head_mean else out

    @staticmethod
    def backward(ctx, grad_out):
        indptr, indices = ctx.adj_sparse
        query, key, x, kept, out = ctx.saved_tensors
        attn, stats = (None, kept) if ctx.stats_only else (kept, None)
        grad_q, grad_k, grad_x = graph_ext.gat_backward(indptr, indices, query, key, x, attn,
                                                        grad_out.contiguous(), out=out,
                                                        head_mean=ctx.head_mean, stats=stats)
        return None, grad_q, grad_k, grad_x, None


def fused_gat(block: block.Block, query: torch.Tensor, key: torch.Tensor, x: torch.Tensor,
              head_mean: bool = False):
    """query [n_dst, H], key [n_src, H], x [n_src, H, F] -> [n_dst, H, F], or
    [n_dst, F] (the mean over heads) with ``head_mean``.

    For a stitched block query is [n_blocks, n_dst, H] and the softmax runs per
    (destination, block tag) like ``fused_gsddmm``'s (sddmm_cuda.cu:11-31): the block is
    taken as ``n_dst * n_blocks`` rows, one per (destination, tag), the fused op runs on
    that view, and the rows of a destination are added up. The tagged rows cost
    ``n_blocks`` output rows per destination instead of one; the attention itself, one
    pass over the edges forward and one backward, is the fused op's."""
    assert x.dim() == 3 and key.dim() == 2
    if query.dim() == 3 and query.size(0) == 1:
        query = query[0]
    if query.dim() == 2:
        return FusedGATFunction.apply(block.adj_sparse, query, key, x, head_mean)
    n_blocks, n_dst = query.size(0), query.size(1)
    view = block.by_query_block(n_blocks)
    per_tag = FusedGATFunction.apply(view.adj_sparse,
                                     query.permute(1, 0, 2).reshape(n_dst * n_blocks, -1), key, x,
                                     head_mean)
    return per_tag.view(n_dst, n_blocks, *per_tag.shape[1:]).sum(dim=1)


class GATHeadsFunction(autograd.Function):
    """A GAT layer's attention stated with per-head attention vectors: query
    ``<a_dst[h], x_dst[n,h,:]>``, key ``<a_src[h], x_src[n,h,:]>``, then the fused
    attention, as one differentiable op. The projections read x once forward; their
    backward is added in place into the gradient the attention already produced for x,
    so x's three uses cost no extra adds."""

    @staticmethod
    def forward(ctx, adj_sparse, x_src, x_dst, a_src, a_dst, head_mean):
        indptr, indices = adj_sparse
        if x_dst is None:
            query, key = graph_ext.head_dot(x_src, a_dst, a_src)
        else:
            query, _ = graph_ext.head_dot(x_dst, a_dst)
            key, _ = graph_ext.head_dot(x_src, a_src)
        ctx.stats_only = graph_ext.gat_one_pass_shape(x_src.size(1), x_src.size(2)) and \
            indices.numel() > 0
        out, attn, *stats = graph_ext.gat_forward(indptr, indices, query, key, x_src,
                                                  stats_only=ctx.stats_only)
        ctx.adj_sparse, ctx.head_mean, ctx.shared = adj_sparse, head_mean, x_dst is None
        saved = (x_src, a_src, a_dst, query, key, stats[0] if ctx.stats_only else attn, out)
        ctx.save_for_backward(*(saved if x_dst is None else saved + (x_dst,)))
        return out.mean(dim=1) if head_mean else out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        indptr, indices = ctx.adj_sparse
        x_src, a_src, a_dst, query, key, kept, out = ctx.saved_tensors[:7]
        attn, stats = (None, kept) if ctx.stats_only else (kept, None)
        grad_q, grad_k, grad_x = graph_ext.gat_backward(
            indptr, indices, query, key, x_src, attn, grad_out.contiguous(), out=out,
            head_mean=ctx.head_mean, stats=stats)
        if ctx.shared:
            grad_x, g_dst, g_src = graph_ext.head_dot_backward(x_src, a_dst, a_src, grad_q, grad_k,
                                                               grad_x=grad_x)
            return None, grad_x, None, g_src, g_dst, None
        x_dst = ctx.saved_tensors[7]
        grad_x, g_src, _ = graph_ext.head_dot_backward(x_src, a_src, None, grad_k, None,
                                                       grad_x=grad_x)
        grad_xd, g_dst, _ = graph_ext.head_dot_backward(x_dst, a_dst, None, grad_q, None)
        return None, grad_x, grad_xd, g_src, g_dst, None


def gat_heads(block: block.Block, x_src: torch.Tensor, a_src: torch.Tensor, a_dst: torch.Tensor,
              x_dst: torch.Tensor = None, head_mean: bool = False):
    """x_src [n_src, H, F] (x_dst [n_dst, H, F] for a bipartite block, default the
    same tensor), a_src / a_dst [H, F] -> [n_dst, H, F], or [n_dst, F] with
    ``head_mean``. Head widths the projection kernels do not take go through
    ``(x * a).sum(-1)`` and ``fused_gat``."""
    assert x_src.dim() == 3 and a_src.shape == a_dst.shape == x_src.shape[1:]
    if graph_ext.head_dot_shape(x_src.size(1), x_src.size(2)):
        return GATHeadsFunction.apply(block.adj_sparse, x_src.contiguous(),
                                      None if x_dst is None else x_dst.contiguous(),
                                      a_src.contiguous(), a_dst.contiguous(), head_mean)
    query = ((x_src if x_dst is None else x_dst) * a_dst).sum(-1)
    key = (x_src * a_src).sum(-1)
    return fused_gat(block, query, key, x_src.contiguous(), head_mean=head_mean)


class EdgeDotFunction(autograd.Function):
    """e[i,h] = <dst[row_i,h,:], src[col_i,h,:]> (dot-product attention logits).
    Backward: grad_dst = SpMM of grad_e with src, grad_src by the transposed gather."""

    @staticmethod
    def forward(ctx, adj_sparse, dst_feat, src_feat):
        indptr, indices = adj_sparse
        ctx.adj_sparse = adj_sparse
        ctx.save_for_backward(dst_feat, src_feat)
        return graph_ext.edge_dot(indptr, indices, dst_feat, src_feat)

    @staticmethod
    def backward(ctx, grad_e):
        indptr, indices = ctx.adj_sparse
        dst_feat, src_feat = ctx.saved_tensors
        grad_e = grad_e.contiguous()
        grad_dst = graph_ext.spmm_forward(grad_e, indptr, indices, src_feat)
        # grad_src[c] = sum_{i: col_i = c} grad_e[i] * dst[row_i]: spmm_backward's grad_x
        # with dst_feat in the role of grad_out
        _, grad_src = graph_ext.spmm_backward(grad_e, indptr, indices, src_feat, dst_feat,
                                              need_grad_a=False)
        return None, grad_dst, grad_src


def edge_dot(block: block.Block, dst_feat: torch.Tensor, src_feat: torch.Tensor):
    return EdgeDotFunction.apply(block.adj_sparse, dst_feat, src_feat)
