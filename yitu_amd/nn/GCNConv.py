"""GCN layer over YiTu_GNN_kernel.forward/backward (YiTu_GNN/nn/GCNConv.py:13-76)."""
import math

import torch as th

from .. import YiTu_GNN_kernel


class GNNAFunction(th.autograd.Function):
    """Saves (X, W) and the inputInfo carrier; backward returns (dX, dW, None)
    (GCNConv.py:13-55). inputInfo needs the attributes row_pointers,
    column_index, degrees, partPtr, part2Node, partSize, dimWorker, warpPerBlock."""

    @staticmethod
    def forward(ctx, X, weight, inputInfo):
        ctx.save_for_backward(X, weight)
        ctx.inputInfo = inputInfo
        ctx.partSize, ctx.dimWorker, ctx.warpPerBlock = (
            inputInfo.partSize, inputInfo.dimWorker, inputInfo.warpPerBlock)
        return YiTu_GNN_kernel.forward(
            X, weight, inputInfo.row_pointers, inputInfo.column_index, inputInfo.degrees,
            inputInfo.partPtr, inputInfo.part2Node, inputInfo.partSize, inputInfo.dimWorker,
            inputInfo.warpPerBlock)[0]

    @staticmethod
    def backward(ctx, d_output):
        X, weight = ctx.saved_tensors
        inputInfo = ctx.inputInfo
        d_input, d_weight = YiTu_GNN_kernel.backward(
            d_output.contiguous(), X, weight, inputInfo.row_pointers, inputInfo.column_index,
            inputInfo.degrees, inputInfo.partPtr, inputInfo.part2Node, ctx.partSize, ctx.dimWorker,
            ctx.warpPerBlock)
        return d_input, d_weight, None


class GCNConv(th.nn.Module):
    """weights ~ U(+-1/sqrt(output_dim)) (GCNConv.py:58-76)."""

    def __init__(self, input_dim, output_dim):
        super().__init__()
        self.weights = th.nn.Parameter(th.randn(input_dim, output_dim))
        self.reset_parameters()

    def reset_parameters(self):
        stdv = 1.0 / math.sqrt(self.weights.size(1))
        self.weights.data.uniform_(-stdv, stdv)

    def forward(self, X, inputInfo):
        return GNNAFunction.apply(X, self.weights, inputInfo)
