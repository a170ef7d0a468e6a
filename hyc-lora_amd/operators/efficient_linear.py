"""Linear layer whose input is saved compressed; the weight gradient is computed straight from the packed codes
by the MFMA kernel.  Reference: operators/efficient_linear.py:11-149."""
import torch

from .. import kernels as K
from ._calibration import CompressionSite, as_rows, fold_statistics
from .compress_function import compress_to_csr, get_statistics


def _linear_backward(grad_output, w, saved, use_bias, needs):
    """(dX, dW, db); `needs` = ctx.needs_input_grad[:3]: a gradient nobody asked for is not computed (a frozen weight
    has no dW, and its input was not saved)"""
    g = grad_output.to(w.dtype)
    grad_input = g @ w if needs[0] else None
    g2, _ = as_rows(g.to(torch.bfloat16))
    grad_weight = None
    if needs[1]:
        # the reference forms [B, out, in] per batch element and lets autograd sum it; here the sum over all tokens
        # is accumulated in fp32 inside the kernel and rounded once
        grad_weight = K.gradw_gemm(g2, saved, out_dtype=torch.float32 if w.dtype == torch.float32 else torch.bfloat16)
        grad_weight = grad_weight.to(w.dtype)
    grad_bias = g2.sum(0).to(w.dtype) if use_bias and needs[2] else None
    return grad_input, grad_weight, grad_bias


class EfficientMemoryLinearFunc(torch.autograd.Function):
    """apply(x, w, b, use_bias, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
    iteration, static_value) -> (x @ w.T (+ b), outlier, L, R, scale)"""

    @staticmethod
    def forward(ctx, x, w, b, use_bias, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method,
                rank, iteration, static_value):
        ctx.use_bias = use_bias
        output = x @ w.transpose(0, 1)
        if use_bias:
            output = output + b[None, ...]
        if iteration < 2:
            outlier, L, R, scale = get_statistics(x, iteration, outlier_ratio, sub_outlier_ratio, sub_outlier_bit,
                                                  sub_outlier_quantize_method, rank)
        else:
            outlier, L, scale, R = static_value[0], static_value[1], static_value[2], static_value[3]
        ctx.saved = None
        if ctx.needs_input_grad[1]:                  # x is kept for dW only
            ctx.saved, _ = compress_to_csr(x, outlier, scale, sub_outlier_bit, sub_outlier_ratio,
                                           L if rank > 0 else None, R if rank > 0 else None)
        ctx.w = w
        ctx.mark_non_differentiable(outlier, L, R, scale)
        return output, outlier, L, R, scale

    @staticmethod
    def backward(ctx, grad_output, grad_outlier, grad_L, grad_R, grad_scale):
        gi, gw, gb = _linear_backward(grad_output, ctx.w.detach(), ctx.saved, ctx.use_bias, ctx.needs_input_grad[:3])
        return gi, gw, gb, None, None, None, None, None, None, None, None


class _ChannelLinearFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, b, plan, bits, group):
        output = x @ w.transpose(0, 1)
        if b is not None:
            output = output + b[None, ...]
        ctx.saved = None
        if ctx.needs_input_grad[1]:                  # x is kept for dW only
            x2, _ = as_rows(x)
            ctx.saved = K.compress_channel(x2, plan, bits, group)
        ctx.w, ctx.use_bias = w, b is not None
        return output

    @staticmethod
    def backward(ctx, grad_output):
        gi, gw, gb = _linear_backward(grad_output, ctx.w.detach(), ctx.saved, ctx.use_bias, ctx.needs_input_grad[:3])
        return gi, gw, gb, None, None, None


class EfficientMemoryLinear(torch.nn.Linear):
    def __init__(self, in_features: int, out_features: int, bias: bool = False, outlier_ratio: float = 0.01,
                 sub_outlier_ratio: float = 0.2, sub_outlier_bit: int = 8, sub_outlier_quantize_method: str = 'per-tensor',
                 rank: int = 16, *, mode: str = "ref", group_size: int = 128, scale_rule: str = "absmax"):
        super(EfficientMemoryLinear, self).__init__(in_features, out_features, bias)
        self.outlier_ratio = outlier_ratio
        self.sub_outlier_ratio = sub_outlier_ratio
        self.sub_outlier_bit = sub_outlier_bit
        self.sub_outlier_quantize_method = sub_outlier_quantize_method
        self.rank = rank
        self.mode = mode
        self.group_size = group_size
        self.site = CompressionSite(outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
                                    mode, group_size, scale_rule)
        self.iteration = 0
        self.static_value = [None, None, None, None]

    def forward(self, input: torch.Tensor):
        if self.mode == "hyc":
            x2, _ = as_rows(input)
            plan = self.site.channel_plan(x2, self.iteration)
            result = _ChannelLinearFunc.apply(input, self.weight, self.bias, plan, self.sub_outlier_bit, self.group_size)
            self.iteration += 1
            return result
        result, outlier, L, R, scale = EfficientMemoryLinearFunc.apply(
            input, self.weight, self.bias, self.bias is not None, self.outlier_ratio, self.sub_outlier_ratio,
            self.sub_outlier_bit, self.sub_outlier_quantize_method, self.rank, self.iteration, self.static_value)
        if self.iteration < 2:
            self.static_value = fold_statistics(self.static_value, self.iteration, outlier, L, scale, R)
        self.iteration += 1
        return result
