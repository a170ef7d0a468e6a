"""RMSNorm whose input is saved compressed.  Forward = one fused kernel (normalise + compress), backward = one
fused kernel (decompress + dx + dw partials) and a column reduce.  Reference: operators/efficient_rmsnorm.py."""
import torch

from .. import kernels as K
from ._calibration import CompressionSite, as_rows, fold_statistics
from .compress_function import get_statistics


def _effective_weight(weight, offset):
    """the weight the kernels multiply by: w, or fp32(w) + 1 for the Gemma form (efficient_rmsnorm_gemma.py:59,100)"""
    w = weight.detach()
    return (w.float() + offset).contiguous() if offset else w.contiguous()


def _ref_forward(ctx, x, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank, weight, eps,
                 iteration, static_value, c2_quirk, weight_offset):
    x = x.contiguous()
    x2, S = as_rows(x)
    if x2.shape[-1] * x.element_size() > 65536:
        raise RuntimeError("This layer norm doesn't support feature dim >= 64KB.")
    if iteration < 2:
        outlier, L, R, scale = get_statistics(x, iteration, outlier_ratio, sub_outlier_ratio, sub_outlier_bit,
                                              sub_outlier_quantize_method, rank)
    else:
        outlier, L, scale, R = static_value[0], static_value[1], static_value[2], static_value[3]
    if sub_outlier_ratio == 0. or sub_outlier_bit == 16:
        raise NotImplementedError("the branches without a quantised part are outside the accelerated path")
    y, rstd, c = K.rmsnorm_fwd_compress_threshold(x2, _effective_weight(weight, weight_offset), eps, S, K.threshold_value(outlier),
                                                  scale.contiguous(), sub_outlier_bit,
                                                  L.contiguous() if rank > 0 else None,
                                                  R.contiguous() if rank > 0 else None, budget=K.kept_budget(outlier))
    ctx.saved = c
    ctx.rstd = rstd
    ctx.weight = weight
    ctx.c2_quirk, ctx.weight_offset = c2_quirk, weight_offset
    ctx.mark_non_differentiable(outlier, L, R, scale)
    return y.reshape(x.shape), outlier, L, R, scale


def _ref_backward(ctx, dy):
    dy2, _ = as_rows(dy.to(torch.bfloat16))
    dx, dw = K.rmsnorm_bwd(dy2, ctx.saved, _effective_weight(ctx.weight, ctx.weight_offset), ctx.rstd, c2_quirk=ctx.c2_quirk)
    return dx.reshape(dy.shape), dw.to(ctx.weight.dtype)


class EfficientMemoryRMSNormFunc(torch.autograd.Function):
    """apply(x, normalized_shape, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
    weight, bias, eps, iteration, static_value) -> (y, outlier, L, R, scale); backward returns dx at slot 0 and dw at
    slot 7 (reference :147-269).  The reference's signature has no room for per-module settings, so this form always
    computes the reference's backward, LayerNorm's mean(w*dy) term included (:102-104); the modules below go through
    _RMSNormFunc, which takes the settings as arguments."""
    weight_offset = 0.0           # 1.0 in the Gemma subclass: a property of the class, never written at run time

    @classmethod
    def forward(cls, ctx, x, normalized_shape, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method,
                rank, weight, bias, eps, iteration, static_value):
        return _ref_forward(ctx, x, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
                            weight, eps, iteration, static_value, True, cls.weight_offset)

    @staticmethod
    def backward(ctx, dy, grad_outlier, grad_L, grad_R, grad_scale):
        dx, dw = _ref_backward(ctx, dy)
        return dx, None, None, None, None, None, None, dw, None, None, None, None


class _RMSNormFunc(torch.autograd.Function):
    """the same operator with the two per-module settings (c2_quirk, weight_offset) as trailing arguments: nothing is
    shared between modules, so modules with different settings can run on different threads"""

    @staticmethod
    def forward(ctx, x, normalized_shape, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method,
                rank, weight, bias, eps, iteration, static_value, c2_quirk, weight_offset):
        return _ref_forward(ctx, x, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
                            weight, eps, iteration, static_value, c2_quirk, weight_offset)

    @staticmethod
    def backward(ctx, dy, grad_outlier, grad_L, grad_R, grad_scale):
        dx, dw = _ref_backward(ctx, dy)
        return dx, None, None, None, None, None, None, dw, None, None, None, None, None, None


class _ChannelRMSNormFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps, plan, bits, group, c2_quirk, weight_offset=0.0):
        x2, _ = as_rows(x)
        y, rstd, c = K.rmsnorm_fwd_compress_channel(x2, _effective_weight(weight, weight_offset), eps, plan, bits, group)
        ctx.saved, ctx.rstd, ctx.weight, ctx.c2_quirk, ctx.weight_offset = c, rstd, weight, c2_quirk, weight_offset
        return y.reshape(x.shape)

    @staticmethod
    def backward(ctx, dy):
        dy2, _ = as_rows(dy.to(torch.bfloat16))
        dx, dw = K.rmsnorm_bwd(dy2, ctx.saved, _effective_weight(ctx.weight, ctx.weight_offset), ctx.rstd,
                               c2_quirk=ctx.c2_quirk)
        return dx.reshape(dy.shape), dw.to(ctx.weight.dtype), None, None, None, None, None, None


class EfficientMemoryRMSNorm(torch.nn.LayerNorm):
    _func = EfficientMemoryRMSNormFunc

    def __init__(self, normalized_shape, eps=1e-05, elementwise_affine=True, bias=True, outlier_ratio: float = 0.01,
                 sub_outlier_ratio: float = 0.2, sub_outlier_bit: int = 8, sub_outlier_quantize_method: str = 'per-tensor',
                 rank: int = 16, *, mode: str = "ref", group_size: int = 128, ref_c2_quirk: bool = True,
                 scale_rule: str = "absmax"):
        super(EfficientMemoryRMSNorm, self).__init__(normalized_shape, eps, elementwise_affine, bias)
        self.outlier_ratio = outlier_ratio
        self.sub_outlier_ratio = sub_outlier_ratio
        self.sub_outlier_bit = sub_outlier_bit
        self.sub_outlier_quantize_method = sub_outlier_quantize_method
        self.rank = rank
        self.mode = mode
        self.group_size = group_size
        self.ref_c2_quirk = ref_c2_quirk
        self.site = CompressionSite(outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
                                    mode, group_size, scale_rule)
        self.iteration = 0
        self.static_value = [None, None, None, None]

    def forward(self, x):
        if self.mode == "hyc":
            x2, _ = as_rows(x)
            plan = self.site.channel_plan(x2, self.iteration)
            y = _ChannelRMSNormFunc.apply(x, self.weight, self.eps, plan, self.sub_outlier_bit, self.group_size,
                                          self.ref_c2_quirk, self._func.weight_offset)
            self.iteration += 1
            return y
        result, outlier, L, R, scale = _RMSNormFunc.apply(
            x, self.normalized_shape, self.outlier_ratio, self.sub_outlier_ratio, self.sub_outlier_bit,
            self.sub_outlier_quantize_method, self.rank, self.weight, self.bias, self.eps, self.iteration,
            self.static_value, self.ref_c2_quirk, self._func.weight_offset)
        if self.iteration < 2:
            self.static_value = fold_statistics(self.static_value, self.iteration, outlier, L, scale, R)
        self.iteration += 1
        return result
