"""Softmax that keeps only the probabilities above a calibrated threshold for its backward.
Reference: operators/efficient_softmax.py:10-75."""
import torch

from .. import kernels as K
from .compress_function import get_statistics_softmax


class EfficientMemorySoftmaxFunc(torch.autograd.Function):
    """apply(x, outlier_ratio, iteration, static_value) -> (softmax(x, -1), outlier)"""

    @staticmethod
    def forward(ctx, x, outlier_ratio, iteration, static_value):
        x = x.contiguous()
        if iteration < 2:
            y, _ = K.softmax_fwd(x)
            outlier = get_statistics_softmax(y, iteration, outlier_ratio)
            ctx.y_sparse = K.softmax_sparsify(y, float(outlier))
        else:
            outlier = static_value
            y, ctx.y_sparse = K.softmax_fwd(x, float(outlier))
        ctx.mark_non_differentiable(outlier)
        return y, outlier

    @staticmethod
    def backward(ctx, grad_output, grad_outlier):
        g = grad_output.to(torch.bfloat16).contiguous()
        return K.softmax_bwd(g, ctx.y_sparse), None, None, None


class EfficientMemorySoftmax(torch.nn.Module):
    def __init__(self, outlier_ratio: float = 0.01):
        super(EfficientMemorySoftmax, self).__init__()
        self.outlier_ratio = outlier_ratio
        self.iteration = 0
        self.static_value = None

    def forward(self, x):
        result, outlier = EfficientMemorySoftmaxFunc.apply(x, self.outlier_ratio, self.iteration, self.static_value)
        if self.iteration < 2:
            self.static_value = (outlier if self.static_value is None
                                 else (self.iteration * self.static_value + outlier) / (self.iteration + 1))
        self.iteration += 1
        return result
