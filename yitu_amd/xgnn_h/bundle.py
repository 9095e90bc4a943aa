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
