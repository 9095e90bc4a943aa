"""GIN layer over YiTu_GNN_kernel.forward_gin/backward_gin (YiTu_GNN/nn/GINConv.py:7-77)."""
import math

import torch

from .. import YiTu_GNN_kernel


class GNNAFunction_GIN(torch.autograd.Function):
    """Saves the aggregate returned by forward_gin together with W
    (GINConv.py:24); backward returns (dX, dW, None, None)."""

    @staticmethod
    def forward(ctx, X, weight, inputInfo, eplison):
        X_prime, X_agg = YiTu_GNN_kernel.forward_gin(
            X, weight, inputInfo.row_pointers, inputInfo.column_index, eplison, inputInfo.partPtr,
            inputInfo.part2Node, inputInfo.partSize, inputInfo.dimWorker, inputInfo.warpPerBlock)
        ctx.save_for_backward(X_agg, weight)
        ctx.inputInfo = inputInfo
        ctx.partSize, ctx.dimWorker, ctx.warpPerBlock, ctx.eplison = (
            inputInfo.partSize, inputInfo.dimWorker, inputInfo.warpPerBlock, eplison)
        return X_prime

    @staticmethod
    def backward(ctx, d_output):
        X, weights = ctx.saved_tensors
        inputInfo = ctx.inputInfo
        d_input, d_weights = YiTu_GNN_kernel.backward_gin(
            d_output.contiguous(), X, weights, inputInfo.row_pointers, inputInfo.column_index,
            ctx.eplison, inputInfo.partPtr, inputInfo.part2Node, ctx.partSize, ctx.dimWorker,
            ctx.warpPerBlock)
        return d_input, d_weights, None, None


class GINConv(torch.nn.Module):
    """epsilon is fixed to 0.5 as in the reference (GINConv.py:62)."""

    def __init__(self, input_dim, output_dim):
        super().__init__()
        self.weights = torch.nn.Parameter(torch.randn(input_dim, output_dim))
        self.eplison = 0.5
        self.reset_parameters()

    def reset_parameters(self):
        stdv = 1.0 / math.sqrt(self.weights.size(1))
        self.weights.data.uniform_(-stdv, stdv)

    def forward(self, X, inputInfo):
        return GNNAFunction_GIN.apply(X, self.weights, inputInfo, self.eplison)
