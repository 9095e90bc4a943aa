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
    ``gspmm(blk, fused_gsddmm(blk, q, k), x)`` as one op, forward and backward."""

    @staticmethod
    def forward(ctx, adj_sparse, query, key, x):
        indptr, indices = adj_sparse
        out, attn = graph_ext.gat_forward(indptr, indices, query, key, x)
        ctx.adj_sparse = adj_sparse
        ctx.save_for_backward(query, key, x, attn, out)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        indptr, indices = ctx.adj_sparse
        query, key, x, attn, out = ctx.saved_tensors
        grad_q, grad_k, grad_x = graph_ext.gat_backward(indptr, indices, query, key, x, attn,
                                                        grad_out.contiguous(), out=out)
        return None, grad_q, grad_k, grad_x


def fused_gat(block: block.Block, query: torch.Tensor, key: torch.Tensor, x: torch.Tensor):
    """query [n_dst, H], key [n_src, H], x [n_src, H, F] -> [n_dst, H, F]."""
    assert x.dim() == 3 and query.dim() == 2 and key.dim() == 2
    return FusedGATFunction.apply(block.adj_sparse, query, key, x)


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
