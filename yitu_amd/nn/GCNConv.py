"""GCN layer over ``YiTu_GNN_kernel.forward / backward`` (the role of
YiTu_GNN/nn/GCNConv.py:13-76)."""
import torch as th

from .. import YiTu_GNN_kernel
from ._common import DenseWeight, graph_arguments


class GNNAFunction(th.autograd.Function):
    """``apply(X, weight, inputInfo)`` -> normalised aggregation of ``X . weight``.
    ``inputInfo`` carries row_pointers, column_index, degrees, partPtr, part2Node,
    partSize, dimWorker, warpPerBlock (GCNConv.py:27-34). Keeps (X, W) for the
    backward, which returns (dX, dW, None)."""

    @staticmethod
    def forward(ctx, X, weight, inputInfo):
        ctx.save_for_backward(X, weight)
        ctx.tail = graph_arguments(inputInfo, inputInfo.degrees)
        # per-edge column scales, when the carrier has prepared them (prepare_edge_scale)
        ctx.edge_scale = getattr(inputInfo, "edge_scale", None)
        return YiTu_GNN_kernel.forward(X, weight, *ctx.tail, edge_scale=ctx.edge_scale)[0]

    @staticmethod
    def backward(ctx, d_output):
        d_input, d_weight = YiTu_GNN_kernel.backward(d_output.contiguous(), *ctx.saved_tensors,
                                                     *ctx.tail, edge_scale=ctx.edge_scale)
        return d_input, d_weight, None


class GCNConv(DenseWeight):
    """``forward(X, inputInfo)`` with ``weights`` [input_dim, output_dim]."""

    def forward(self, X, inputInfo):
        return GNNAFunction.apply(X, self.weights, inputInfo)
