"""GIN layer over ``YiTu_GNN_kernel.forward_gin / backward_gin`` (the role of
YiTu_GNN/nn/GINConv.py)."""
import torch

from .. import YiTu_GNN_kernel
from ._common import DenseWeight, graph_arguments


class GNNAFunction_GIN(torch.autograd.Function):
    """``apply(X, weight, inputInfo, eplison)`` -> ``(eplison * sum of neighbours) . weight``.
    The aggregate that ``forward_gin`` returns beside the output is what the
    backward needs in place of X (GINConv.py:24), so X itself is not kept.
    Gradients: (dX, dW, None, None)."""

    @staticmethod
    def forward(ctx, X, weight, inputInfo, eplison):
        tail = graph_arguments(inputInfo, eplison)
        out, aggregate = YiTu_GNN_kernel.forward_gin(X, weight, *tail)
        ctx.save_for_backward(aggregate, weight)
        ctx.tail = tail
        return out

    @staticmethod
    def backward(ctx, d_output):
        aggregate, weight = ctx.saved_tensors
        d_input, d_weight = YiTu_GNN_kernel.backward_gin(d_output.contiguous(), aggregate, weight,
                                                         *ctx.tail)
        return d_input, d_weight, None, None


class GINConv(DenseWeight):
    """``forward(X, inputInfo)``; the neighbour sum is scaled by ``eplison`` = 0.5,
    a constant of the layer as in the reference (GINConv.py:62)."""

    def __init__(self, input_dim, output_dim):
        super().__init__(input_dim, output_dim)
        self.eplison = 0.5

    def forward(self, X, inputInfo):
        return GNNAFunction_GIN.apply(X, self.weights, inputInfo, self.eplison)
