"""EfficientMemorySiLU / EfficientMemoryGELU share everything except the activation; see efficient_gelu.py.
Reference: operators/efficient_silu.py:11-113."""
import torch
import torch.nn.functional as F

from .. import kernels as K
from ._calibration import CompressionSite, as_rows, fold_statistics
from .compress_function import compress_to_csr, get_statistics, head_to_hidden_shape, hidden_to_head_shape


def _ref_forward(ctx, x, act_fwd, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, method, rank, iteration, static_value):
    result = act_fwd(x)
    if iteration < 2:
        outlier, L, R, scale = get_statistics(x, iteration, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, method, rank)
    else:
        outlier, L, scale, R = static_value[0], static_value[1], static_value[2], static_value[3]
    ctx.saved, ctx.hidden_shape = compress_to_csr(x, outlier, scale, sub_outlier_bit, sub_outlier_ratio,
                                                  L if rank > 0 else None, R if rank > 0 else None)
    ctx.is_head = x.dim() == 4
    ctx.num_heads = x.shape[1] if ctx.is_head else 1
    ctx.mark_non_differentiable(outlier, L, R, scale)
    return result, outlier, L, R, scale


def _ref_backward(ctx, act, grad_output):
    g = grad_output.to(torch.bfloat16)
    if ctx.is_head:
        g = head_to_hidden_shape(g)
    g2, _ = as_rows(g)
    dx = K.act_bwd(act, g2, ctx.saved).reshape(ctx.hidden_shape)
    if ctx.is_head:
        dx = hidden_to_head_shape(dx, ctx.num_heads)
    return dx


class EfficientMemorySiLUFunc(torch.autograd.Function):
    """apply(x, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank, iteration,
    static_value) -> (silu(x), outlier, L, R, scale); x is saved as INT codes + sparse outliers."""

    @staticmethod
    def forward(ctx, x, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
                iteration, static_value):
        return _ref_forward(ctx, x, F.silu, outlier_ratio, sub_outlier_ratio, sub_outlier_bit,
                            sub_outlier_quantize_method, rank, iteration, static_value)

    @staticmethod
    def backward(ctx, grad_output, grad_outlier, grad_L, grad_R, grad_scale):
        return _ref_backward(ctx, "silu", grad_output), None, None, None, None, None, None, None


class _ChannelActFunc(torch.autograd.Function):
    """channel-mode twin: apply(x, act, plan, bits, group) -> act(x); x saved as ChannelCompressed"""

    @staticmethod
    def forward(ctx, x, act, plan, bits, group):
        x2, _ = as_rows(x)
        ctx.act = act
        if K.act_fwd_compress_supported(x2.shape[-1], bits, group):
            y, ctx.saved = K.act_fwd_compress(act, x2, plan, bits, group)      # one read of x
            return y.view(x.shape)
        ctx.saved = K.compress_channel(x2, plan, bits, group)
        return F.silu(x) if act == "silu" else F.gelu(x)

    @staticmethod
    def backward(ctx, grad_output):
        g2, _ = as_rows(grad_output.to(torch.bfloat16))
        return K.act_bwd(ctx.act, g2, ctx.saved).reshape(grad_output.shape), None, None, None, None


class _ActModule(torch.nn.Module):
    _act = "silu"
    _func = EfficientMemorySiLUFunc

    def __init__(self, outlier_ratio: float = 0.01, sub_outlier_ratio: float = 0.2, sub_outlier_bit: int = 8,
                 sub_outlier_quantize_method: str = 'per-tensor', rank: int = 16, *, mode: str = "ref",
                 group_size: int = 128, scale_rule: str = "absmax"):
        super().__init__()
        self.site = CompressionSite(outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method,
                                    rank, mode, group_size, scale_rule)
        self.outlier_ratio = outlier_ratio
        self.sub_outlier_ratio = sub_outlier_ratio
        self.sub_outlier_bit = sub_outlier_bit
        self.sub_outlier_quantize_method = sub_outlier_quantize_method
        self.rank = rank
        self.mode = mode
        self.group_size = group_size
        self.iteration = 0
        self.static_value = [None, None, None, None]

    def forward(self, input):
        if self.mode == "hyc":
            x2, _ = as_rows(input)
            plan = self.site.channel_plan(x2, self.iteration)
            result = _ChannelActFunc.apply(input, self._act, plan, self.sub_outlier_bit, self.group_size)
            self.iteration += 1
            return result
        result, outlier, L, R, scale = self._func.apply(
            input, self.outlier_ratio, self.sub_outlier_ratio, self.sub_outlier_bit, self.sub_outlier_quantize_method,
            self.rank, self.iteration, self.static_value)
        if self.iteration < 2:
            self.static_value = fold_statistics(self.static_value, self.iteration, outlier, L, scale, R)
        self.iteration += 1
        return result


class EfficientMemorySiLU(_ActModule):
    _act = "silu"
    _func = EfficientMemorySiLUFunc
