"""Autograd glue over the graph_ext ops (xgnn_h/sparse.py), unchanged in
behaviour: same Function classes, saved tensors, asserts and gradients."""
import torch
from torch import autograd

from .. import graph_ext
from . import block


class GSPMMFunction(autograd.Function):
    """sparse.py:7-35"""

    @staticmethod
    def forward(ctx, adj_sparse, adj_values, x):
        indptr, indices = adj_sparse[0], adj_sparse[1]
        y = graph_ext.spmm_forward(adj_values, indptr, indices, x)
        ctx.adj_sparse = adj_sparse
        ctx.save_for_backward(adj_values, x)
        return y

    @staticmethod
    def backward(ctx, grad_out):
        indptr, indices = ctx.adj_sparse[0], ctx.adj_sparse[1]
        values, x = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        assert len(ctx.needs_input_grad) == 3
        assert ctx.needs_input_grad[0] is False
        # a gradient nobody asked for (constant edge weights) is not computed
        grad_a, grad_x = graph_ext.spmm_backward(values, indptr, indices, x, grad_out,
                                                 need_grad_a=ctx.needs_input_grad[1],
                                                 need_grad_x=ctx.needs_input_grad[2])
        return None, grad_a, grad_x


def gspmm(block: block.Block, edge: torch.Tensor, x: torch.Tensor):
    """sparse.py:38-51: ``edge=None`` aggregates with unit weights."""
    assert x.dim() == 3
    indices = block.adj_sparse[1]
    if edge is None:
        edge = torch.ones(size=[indices.size(0), x.size(1)], device=x.device)
    return GSPMMFunction.apply(block.adj_sparse, edge, x)


class GSDDMMFunction(autograd.Function):
    """sparse.py:54-81"""

    @staticmethod
    def forward(ctx, adj_sparse, query, key):
        indptr, indices = adj_sparse
        attn_values = graph_ext.sddmm_forward(indptr, indices, query, key)
        ctx.adj_sparse = adj_sparse
        ctx.save_for_backward(query, key, attn_values)
        return attn_values

    @staticmethod
    def backward(ctx, grad_out):
        grad_out = grad_out.contiguous()
        indptr, indices = ctx.adj_sparse
        query, key, attn_values = ctx.saved_tensors
        assert len(ctx.needs_input_grad) == 3
        assert ctx.needs_input_grad[0] is False
        assert ctx.needs_input_grad[1] is True
        assert ctx.needs_input_grad[2] is True
        grad_query, grad_key = graph_ext.sddmm_backward(indptr, indices, query, key, attn_values,
                                                        grad_out)
        return None, grad_query, grad_key


def fused_gsddmm(block: block.Block, query: torch.Tensor, key: torch.Tensor):
    """sparse.py:84-91"""
    if query.dim() == 2:
        query = query.unsqueeze(0)
    return GSDDMMFunction.apply(block.adj_sparse, query, key)


class HFUSEDFunction(autograd.Function):
    """sparse.py:94-110, with the backward the reference leaves unimplemented."""

    @staticmethod
    def forward(ctx, spmm_sparse, spmm_values, spmm_x, sddmm_sparse, sddmm_query, sddmm_key):
        spmm_out, attn_values = graph_ext.hfused_forward(
            spmm_values, spmm_sparse[0], spmm_sparse[1], spmm_x,
            sddmm_sparse[0], sddmm_sparse[1], sddmm_query, sddmm_key)
        ctx.spmm_sparse = spmm_sparse
        ctx.sddmm_sparse = sddmm_sparse
        ctx.save_for_backward(spmm_values, spmm_x, sddmm_query, sddmm_key, attn_values)
        return spmm_out, attn_values

    @staticmethod
    def backward(ctx, grad_spmm, grad_attn):
        spmm_values, spmm_x, sddmm_query, sddmm_key, attn_values = ctx.saved_tensors
        grad_a, grad_x, grad_q, grad_k = graph_ext.hfused_backward(
            spmm_values, ctx.spmm_sparse[0], ctx.spmm_sparse[1], spmm_x, grad_spmm.contiguous(),
            ctx.sddmm_sparse[0], ctx.sddmm_sparse[1], sddmm_query, sddmm_key, attn_values,
            grad_attn.contiguous())
        return None, grad_a, grad_x, None, grad_q, grad_k


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
        ctx.save_for_backward(query, key, x, attn)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        indptr, indices = ctx.adj_sparse
        query, key, x, attn = ctx.saved_tensors
        grad_q, grad_k, grad_x = graph_ext.gat_backward(indptr, indices, query, key, x, attn,
                                                        grad_out.contiguous())
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
        _, grad_src = graph_ext.spmm_backward(grad_e, indptr, indices, src_feat, dst_feat)
        return None, grad_dst, grad_src


def edge_dot(block: block.Block, dst_feat: torch.Tensor, src_feat: torch.Tensor):
    return EdgeDotFunction.apply(block.adj_sparse, dst_feat, src_feat)
