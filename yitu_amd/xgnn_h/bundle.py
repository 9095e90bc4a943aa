"""Two Linear layers that read one input, as a single grouped GEMM launch
(the role of xgnn_h/bundle.py)."""
from torch import autograd
from torch.autograd.function import once_differentiable

from .. import graph_ext


class GEMMBundleFunction(autograd.Function):
    """``(x w_1^T, x w_2^T)`` from one launch of the grouped MFMA GEMM, and its
    backward ``(dx, dw_1, dw_2)`` from ``graph_ext.b2gemm_backward``.

    Call signature as in bundle.py:6-26: ``apply(x, w_1, w_2, b_1, b_2)``. The two
    bias arguments take no part in the product and receive no gradient, exactly
    as there; a caller that wants biases adds them to the results.
    """

    @staticmethod
    def forward(ctx, x, w_1, w_2, b_1=None, b_2=None):
        ctx.save_for_backward(x, w_1, w_2)
        return tuple(graph_ext.b2gemm(x, w_1, w_2))

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_1, grad_2):
        grads = graph_ext.b2gemm_backward(*ctx.saved_tensors, grad_1.contiguous(),
                                          grad_2.contiguous())
        return (*grads, None, None)


class SkinnyLinearFunction(autograd.Function):
    """``F.linear(x, weight, bias)`` for a handful of output features (the query / key
    projections of a GAT layer): one read of x forward; backward reads x once and writes
    grad_x once."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        return graph_ext.skinny_linear(x, weight, bias)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_y):
        x, weight = ctx.saved_tensors
        grad_x, grad_w, grad_b = graph_ext.skinny_linear_backward(
            x, weight, grad_y.contiguous(), need_bias=ctx.has_bias)
        return grad_x, grad_w, grad_b


class LinearPairFunction(autograd.Function):
    """``(x w_a^T + b_a, x w_b^T + b_b)``: the grouped product of ``GEMMBundleFunction`` with
    the biases inside, their gradients as the library's fixed-order column sums (torch's own
    reduction clears an accumulator with a memset node, which does not replay reliably from
    a captured HIP graph)."""

    @staticmethod
    def forward(ctx, x, w_a, w_b, b_a, b_b):
        ctx.save_for_backward(x, w_a, w_b)
        y_a, y_b = graph_ext.b2gemm(x, w_a, w_b)
        if b_a is not None:
            y_a.add_(b_a)
        if b_b is not None:
            y_b.add_(b_b)
        return y_a, y_b

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_a, grad_b):
        grad_a, grad_b = grad_a.contiguous(), grad_b.contiguous()
        dx, dw_a, dw_b = graph_ext.b2gemm_backward(*ctx.saved_tensors, grad_a, grad_b)
        db_a = graph_ext.column_sum(grad_a) if ctx.needs_input_grad[3] else None
        db_b = graph_ext.column_sum(grad_b) if ctx.needs_input_grad[4] else None
        return dx, dw_a, dw_b, db_a, db_b


def bundled_linear(x, w_a, w_b, b_a=None, b_b=None):
    """``(x w_a^T + b_a, x w_b^T + b_b)`` for two weight matrices of equal shape applied
    to one 2-D input: with a handful of outputs one skinny product over the stacked
    weights (one read of x), otherwise the grouped GEMM launch plus the biases."""
    import torch
    n_out = w_a.size(0)
    if (b_a is None) == (b_b is None) and x.dtype == torch.float32 and \
            graph_ext.skinny_linear_shape(w_a.size(1), 2 * n_out):
        bias = None if b_a is None else torch.cat([b_a, b_b])
        y = SkinnyLinearFunction.apply(x.contiguous(), torch.cat([w_a, w_b], dim=0), bias)
        return y[:, :n_out].contiguous(), y[:, n_out:].contiguous()
    if b_a is None and b_b is None:
        return GEMMBundleFunction.apply(x, w_a, w_b, None, None)
    return LinearPairFunction.apply(x, w_a, w_b, b_a, b_b)


def linear_pair(x, linear_a, linear_b):
    """``(linear_a(x), linear_b(x))`` for two ``nn.Linear`` that read the same input."""
    if x.dim() == 2 and x.is_cuda and linear_a.weight.shape == linear_b.weight.shape and \
            linear_a.weight.stride() == linear_b.weight.stride():
        return bundled_linear(x, linear_a.weight, linear_b.weight, linear_a.bias, linear_b.bias)
    return linear_a(x), linear_b(x)


class MfmaLinearFunction(autograd.Function):
    """``F.linear(x, weight, bias)`` on the library's fp32 MFMA GEMM: ``x . weight^T`` and both
    gradient products at the same rate whatever the operand layout, the bias gradient as
    a fixed-order column sum."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        return graph_ext.linear_forward(x, weight, None if bias is None else bias.contiguous())

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_y):
        x, weight = ctx.saved_tensors
        grad_y = grad_y.contiguous()
        grad_x = graph_ext.sgemm(grad_y, weight) if ctx.needs_input_grad[0] else None
        grad_w = graph_ext.sgemm(grad_y, x, trans_a=True) if ctx.needs_input_grad[1] else None
        grad_b = graph_ext.column_sum(grad_y) if ctx.has_bias and ctx.needs_input_grad[2] else None
        return grad_x, grad_w, grad_b


def linear(x, weight, bias=None):
    """``F.linear`` for 2-D fp32 device tensors on the library's kernels: the skinny product
    for a handful of outputs, the MFMA GEMM otherwise; anything else goes to torch."""
    import torch
    from torch.nn import functional as F
    if x.dim() == 2 and x.is_cuda and x.dtype == torch.float32 and weight.dtype == torch.float32 \
            and x.size(0) > 0:
        if graph_ext.skinny_linear_shape(weight.size(1), weight.size(0)):
            return SkinnyLinearFunction.apply(x.contiguous(), weight.contiguous(), bias)
        return MfmaLinearFunction.apply(x.contiguous(), weight.contiguous(), bias)
    return F.linear(x, weight, bias)
