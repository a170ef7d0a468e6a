"""Softmax over the last dimension whose backward runs from the few probabilities above a calibrated threshold.

Mirror of the reference's operators/efficient_softmax.py:10-75 (same class names, `apply` signature, `iteration` /
`static_value` attributes).  Steady state is one kernel for y plus the per-row counts of kept entries, one for the row
offsets and one that writes the kept entries as CSR (int32 column, bf16 value), with no host round trip from the
second steady-state call on (kernels.KeptBudget); the backward reads the incoming gradient once:
dx = (g - sum_j g_j * p_j) * p with p zero outside the kept set.
"""
import torch

from .. import kernels as K
from ._calibration import running_mean
from .compress_function import get_statistics_softmax

_CALIBRATION_CALLS = 2      # the threshold is measured on the first two calls and frozen afterwards


class EfficientMemorySoftmaxFunc(torch.autograd.Function):
    """apply(x, outlier_ratio, iteration, static_value) -> (softmax(x, -1), threshold)"""

    @staticmethod
    def forward(ctx, x, outlier_ratio, iteration, static_value):
        scores = x.contiguous()
        if iteration >= _CALIBRATION_CALLS:
            threshold = static_value
            probs, ctx.kept = K.softmax_fwd(scores, K.threshold_value(threshold), budget=K.kept_budget(threshold))
        else:
            # the threshold of this call comes from its own probabilities, so they are needed before the pruning
            probs, _ = K.softmax_fwd(scores)
            threshold = get_statistics_softmax(probs, iteration, outlier_ratio)
            ctx.kept = K.softmax_sparsify(probs, K.threshold_value(threshold))
        ctx.mark_non_differentiable(threshold)
        return probs, threshold

    @staticmethod
    def backward(ctx, grad_probs, _grad_threshold):
        return K.softmax_bwd(grad_probs.to(torch.bfloat16).contiguous(), ctx.kept), None, None, None


class EfficientMemorySoftmax(torch.nn.Module):
    def __init__(self, outlier_ratio: float = 0.01):
        super().__init__()
        self.outlier_ratio = outlier_ratio
        self.iteration = 0
        self.static_value = None

    def forward(self, x):
        probs, threshold = EfficientMemorySoftmaxFunc.apply(x, self.outlier_ratio, self.iteration, self.static_value)
        if self.iteration < _CALIBRATION_CALLS:
            self.static_value = running_mean(self.static_value, threshold, self.iteration)
        self.iteration += 1
        return probs
