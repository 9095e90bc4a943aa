"""Time encoding and the temporal attention layer (YiTu_GNN/YiTu_T/layers.py:6-17,
39-142) without DGL: the message-flow block is the sampler's COO output, the
edge softmax / weighted sum run on the graph_ext kernels.

The reference computes the attention core with DGL ops that are not part of its
own tree (dgl.ops.edge_softmax, update_all(copy_src, sum), layers.py:131-135);
their arithmetic is restated here as
    logits = sum_d Q[dst] * K[e]          (per-edge dot, H heads)
    att    = softmax over each destination's edges of LeakyReLU_0.2(logits)
    agg    = sum_e att[e] * V[e]
"""
import numpy as np
import torch

from .. import graph_ext
from . import fused
from ..xgnn_h import block as xblock
from ..xgnn_h import bundle, sparse


def _linear(layer: torch.nn.Linear, x):
    """``layer(x)`` on the library's GEMM, with the bias gradient as a fixed-order column
    sum: at these sizes (a few thousand rows, 100 to 272 columns) the products are several
    times faster than the BLAS library's choice of kernel, and torch's own bias reduction
    records a memset node that does not replay reliably from a captured HIP graph, so with
    this the whole training step of the layer can be captured."""
    if x.is_cuda and x.dtype == torch.float32 and x.dim() == 2:
        return bundle.linear(x, layer.weight, layer.bias)
    return layer(x)


class _DotAttentionFunction(torch.autograd.Function):
    """agg[r] = sum_e softmax_r(LeakyReLU_0.2(<Q[r], K[e]>)) V[e] over a block whose edge e
    has its own source row e: ``sparse.edge_dot`` -> ``sparse.fused_gsddmm`` (zero query,
    the logits as per-edge keys) -> ``sparse.gspmm`` on the same kernels, as one autograd
    node (each node costs more host time than its kernels take at these sizes)."""

    @staticmethod
    def forward(ctx, adj_sparse, Q, K, V):
        indptr, indices = adj_sparse
        logits = graph_ext.edge_dot(indptr, indices, Q, K)
        zeros = torch.zeros((1, Q.size(0), Q.size(1)), device=Q.device)
        att = graph_ext.sddmm_forward(indptr, indices, zeros, logits)
        ctx.adj_sparse = adj_sparse
        ctx.save_for_backward(Q, K, V, logits, att, zeros)
        return graph_ext.spmm_forward(att, indptr, indices, V)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_agg):
        indptr, indices = ctx.adj_sparse
        Q, K, V, logits, att, zeros = ctx.saved_tensors
        grad_att, grad_v = graph_ext.spmm_backward(att, indptr, indices, V, grad_agg.contiguous())
        _, grad_logits = graph_ext.sddmm_backward(indptr, indices, zeros, logits, att, grad_att)
        grad_q = graph_ext.spmm_forward(grad_logits, indptr, indices, K)
        _, grad_k = graph_ext.spmm_backward(grad_logits, indptr, indices, K, Q, need_grad_a=False)
        return None, grad_q, grad_k, grad_v


class TimeEncode(torch.nn.Module):
    """cos(t * w + b), w_i = 10^(-9 i / (dim - 1)), b = 0, both trainable (layers.py:6-17)."""

    def __init__(self, dim):
        super().__init__()
        self.dim = dim
        self.w = torch.nn.Linear(1, dim)
        self.w.weight = torch.nn.Parameter(
            torch.from_numpy(1 / 10 ** np.linspace(0, 9, dim, dtype=np.float32)).reshape(dim, -1))
        self.w.bias = torch.nn.Parameter(torch.zeros(dim))

    def forward(self, t):
        return torch.cos(_linear(self.w, t.reshape((-1, 1))))


class TemporalBlock:
    """What the layer needs of a sampled block: ``n_dst`` roots, edges sorted by
    root slot, one new source node per edge (as sampler_core emits them).
    ``h`` holds the node features [n_dst + n_edges, dim_node_feat] (roots first),
    ``dt`` the per-edge time deltas, ``f`` optional edge features."""

    def __init__(self, row, n_dst, dt, h=None, f=None, device="cuda"):
        dev = torch.device(device)
        row = torch.as_tensor(np.asarray(row), dtype=torch.int64)
        if row.numel() and not bool((row[1:] >= row[:-1]).all()):
            raise ValueError("edges must be grouped by destination (ascending root slot)")
        counts = torch.bincount(row, minlength=n_dst)
        indptr = torch.zeros(n_dst + 1, dtype=torch.int64)
        indptr[1:] = torch.cumsum(counts, 0)
        self.n_dst = int(n_dst)
        self.n_edges = int(row.numel())
        self.row = row.to(dev)
        self.blk = xblock.Block([n_dst, self.n_edges],
                                [indptr.to(torch.int32),
                                 torch.arange(self.n_edges, dtype=torch.int32)]).to(dev)
        self.dt = torch.as_tensor(np.asarray(dt), dtype=torch.float32).to(dev)
        self.h = h
        self.f = f

    @staticmethod
    def from_sampler(tgb, memory=None, device="cuda"):
        """Builds the block from a ``TemporalGraphBlock`` and gathers node features
        from a ``[num_nodes, dim]`` table by node id (the reference's prepare_input)."""
        n_dst = tgb.dim_out()
        h = None
        if memory is not None:
            ids = torch.as_tensor(tgb.nodes(), dtype=torch.int64, device=memory.device)
            h = memory[ids].to(device)
        return TemporalBlock(tgb.row(), n_dst, tgb.dts()[n_dst:], h=h, device=device)

    @staticmethod
    def from_device_block(dtgb, memory):
        """The same from a DeviceTemporalGraphBlock (GpuParallelSampler): nothing
        leaves the GPU. ``memory`` is the [num_nodes, dim] feature table on it."""
        b = TemporalBlock.__new__(TemporalBlock)
        dev = memory.device
        n_dst = dtgb.dim_out()
        row = dtgb.row().to(torch.int64)
        indptr = torch.zeros(n_dst + 1, dtype=torch.int64, device=dev)
        indptr[1:] = torch.cumsum(torch.bincount(row, minlength=n_dst), 0)
        b.n_dst = int(n_dst)
        b.n_edges = int(row.numel())
        b.row = row
        b.blk = xblock.Block([n_dst, b.n_edges],
                             [indptr.to(torch.int32),
                              torch.arange(b.n_edges, dtype=torch.int32, device=dev)])
        b.dt = dtgb.dts()[n_dst:]
        b.h = memory[dtgb.nodes().to(torch.int64)]
        b.f = None
        return b

    def num_edges(self):
        return self.n_edges

    def num_dst_nodes(self):
        return self.n_dst


class TransfomerAttentionLayer(torch.nn.Module):
    """layers.py:39-142. Parameter names and shapes are the reference's, so its
    state_dicts load unchanged. ``combined=True`` (layers.py:53-66, 81-103) keeps one
    Linear per input part (node / edge / time) and adds their results; that is the
    product of the concatenated inputs with the concatenated weights, biases added up,
    which is how it is computed here (same kernels as the other branch)."""

    def __init__(self, dim_node_feat, dim_edge_feat, dim_time, num_head, dropout, att_dropout,
                 dim_out, combined=False):
        super().__init__()
        self.combined = combined
        self.num_head = num_head
        self.dim_node_feat = dim_node_feat
        self.dim_edge_feat = dim_edge_feat
        self.dim_time = dim_time
        self.dim_out = dim_out
        self.dropout = torch.nn.Dropout(dropout)
        self.att_dropout = torch.nn.Dropout(att_dropout)
        self.att_act = torch.nn.LeakyReLU(0.2)
        if dim_time > 0:
            self.time_enc = TimeEncode(dim_time)
        if combined:
            if dim_node_feat > 0:
                self.w_q_n = torch.nn.Linear(dim_node_feat, dim_out)
                self.w_k_n = torch.nn.Linear(dim_node_feat, dim_out)
                self.w_v_n = torch.nn.Linear(dim_node_feat, dim_out)
            if dim_edge_feat > 0:
                self.w_k_e = torch.nn.Linear(dim_edge_feat, dim_out)
                self.w_v_e = torch.nn.Linear(dim_edge_feat, dim_out)
            if dim_time > 0:
                self.w_q_t = torch.nn.Linear(dim_time, dim_out)
                self.w_k_t = torch.nn.Linear(dim_time, dim_out)
                self.w_v_t = torch.nn.Linear(dim_time, dim_out)
        else:
            if dim_node_feat + dim_time > 0:
                self.w_q = torch.nn.Linear(dim_node_feat + dim_time, dim_out)
            self.w_k = torch.nn.Linear(dim_node_feat + dim_edge_feat + dim_time, dim_out)
            self.w_v = torch.nn.Linear(dim_node_feat + dim_edge_feat + dim_time, dim_out)
        self.w_out = torch.nn.Linear(dim_node_feat + dim_out, dim_out)
        self.layer_norm = torch.nn.LayerNorm(dim_out)

    def _projection(self, which):
        """(weight, bias) of the q / k / v projection over the concatenated inputs
        [node | edge | time] (q: [node | time]); None when q has no input."""
        if not self.combined:
            lin = getattr(self, "w_" + which, None)
            return (lin.weight, lin.bias) if lin is not None else None
        parts = [getattr(self, "w_%s_%s" % (which, tag), None)
                 for tag, dim in (("n", self.dim_node_feat), ("e", self.dim_edge_feat),
                                  ("t", self.dim_time)) if dim > 0 and not (which == "q" and tag == "e")]
        parts = [p for p in parts if p is not None]
        if not parts:
            return None
        weight = parts[0].weight if len(parts) == 1 else torch.cat([p.weight for p in parts], dim=1)
        bias = parts[0].bias
        for p in parts[1:]:
            bias = bias + p.bias
        return weight, bias

    def forward(self, b: TemporalBlock):
        assert self.dim_time + self.dim_node_feat + self.dim_edge_feat > 0
        dev = self.w_out.weight.device
        wq, wk, wv = self._projection("q"), self._projection("k"), self._projection("v")
        n_dst = b.num_dst_nodes()
        if b.num_edges() == 0:
            return torch.zeros((n_dst, self.dim_out), device=dev)
        drops = self.training and (self.dropout.p > 0 or self.att_dropout.p > 0)
        if not drops and wk[0].is_cuda and wk[0].dtype == torch.float32 and \
                fused.supported(self.dim_node_feat, self.dim_edge_feat, self.dim_time, self.dim_out,
                                self.num_head):
            # the whole layer as one autograd node of twelve launches
            te = self.time_enc.w if self.dim_time > 0 else None
            return fused.TemporalAttentionFunction.apply(
                b.blk.adj_sparse[0], n_dst, self.num_head, self.layer_norm.eps,
                b.h if self.dim_node_feat > 0 else None, b.f if self.dim_edge_feat > 0 else None,
                b.dt, te.weight if te is not None else None, te.bias if te is not None else None,
                wq[0], wq[1], wk[0], wk[1], wv[0], wv[1], self.w_out.weight, self.w_out.bias,
                self.layer_norm.weight, self.layer_norm.bias)
        parts_q, parts_kv = [], []
        if self.dim_node_feat > 0:
            parts_q.append(b.h[:n_dst])
            parts_kv.append(b.h[n_dst:])
        if self.dim_edge_feat > 0:
            parts_kv.append(b.f)
        if self.dim_time > 0:
            parts_kv.append(self.time_enc(b.dt))
            parts_q.append(self.time_enc(torch.zeros(n_dst, dtype=torch.float32, device=dev)))
        kv_in = torch.cat(parts_kv, dim=1)
        head_dim = self.dim_out // self.num_head
        if parts_q:
            Q = bundle.linear(torch.cat(parts_q, dim=1), wq[0], wq[1])
        elif self.combined:  # nothing is added to the zeros Q starts from (layers.py:82)
            Q = torch.zeros((n_dst, self.dim_out), device=dev)
        else:  # edge features only (layers.py:104-107)
            Q = torch.ones((n_dst, self.dim_out), device=dev)
        K, V = bundle.bundled_linear(kv_in, wk[0], wv[0], wk[1], wv[1])  # one grouped launch
        K = K.reshape(-1, self.num_head, head_dim).contiguous()
        V = V.reshape(-1, self.num_head, head_dim).contiguous()
        Q = Q.reshape(n_dst, self.num_head, head_dim).contiguous()
        # att = edge_softmax(LeakyReLU(sum_d Q*K)); fused_gsddmm applies LeakyReLU(0.2) +
        # softmax to (query + key): query = 0, key = the dot-product logits, one key per edge
        if self.training and self.att_dropout.p > 0:
            logits = sparse.edge_dot(b.blk, Q, K)
            zeros = torch.zeros((n_dst, self.num_head), device=dev)
            att = sparse.fused_gsddmm(b.blk, zeros.requires_grad_(), logits)
            agg = sparse.gspmm(b.blk, self.att_dropout(att), V)
        else:
            agg = _DotAttentionFunction.apply(b.blk.adj_sparse, Q, K, V)
        agg = agg.reshape(n_dst, self.dim_out)
        rst = torch.cat([agg, b.h[:n_dst]], dim=1) if self.dim_node_feat != 0 else agg
        rst = _linear(self.w_out, rst)
        rst = torch.nn.functional.relu(self.dropout(rst))
        return self.layer_norm(rst)
