"""GELU with the compressed input saved for backward.  Forward is the exact (erf) GELU, backward the tanh-form
derivative, as in the reference: operators/efficient_gelu.py:11-124."""
import torch
import torch.nn.functional as F

from .efficient_silu import _ActModule, _ref_backward, _ref_forward


class EfficientMemoryGELUFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
                iteration, static_value):
        return _ref_forward(ctx, x, F.gelu, outlier_ratio, sub_outlier_ratio, sub_outlier_bit,
                            sub_outlier_quantize_method, rank, iteration, static_value)

    @staticmethod
    def backward(ctx, grad_output, grad_outlier, grad_L, grad_R, grad_scale):
        return _ref_backward(ctx, "gelu", grad_output), None, None, None, None, None, None, None


class EfficientMemoryGELU(_ActModule):
    _act = "gelu"
    _func = EfficientMemoryGELUFunc
