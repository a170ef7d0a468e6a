"""LayerNorm whose input is saved compressed.  Reference: operators/efficient_layernorm.py (forward kernel :15-61,
backward :66-148, Function :203-330, module :333-405).

The forward is one kernel (statistics, y and the compressed x from a single read of x, the RMSNorm forward kernel
with the row mean added); the backward is the fused decompress + dx + dw kernel of the RMSNorm path with the row mean
folded in (xn = (x_hat - mean) * rstd), and db = sum of dy.  Rows too long for the one-pass forward (more than 1024
chunks per segment) take the framework's layer norm followed by the compress kernel."""
import torch

from .. import kernels as K
from ._calibration import CompressionSite, as_rows, fold_statistics
from .compress_function import compress_to_csr, get_statistics


def _forward_stats(x2, weight, bias, eps):
    if weight.dtype != x2.dtype:                        # fp32 norm weights on bf16 activations: evaluate in fp32
        b32 = bias.float() if bias is not None else None
        y, mean, rstd = torch.native_layer_norm(x2.float(), (x2.shape[-1],), weight.float(), b32, eps)
        y = y.to(x2.dtype)
    else:
        y, mean, rstd = torch.native_layer_norm(x2, (x2.shape[-1],), weight, bias, eps)
    return y, mean.reshape(-1).float().contiguous(), rstd.reshape(-1).float().contiguous()


def _affine(weight, bias):
    """(w, b) as the kernels read them: contiguous, the bias in the weight's dtype"""
    w = weight.detach().contiguous()
    b = None if bias is None else bias.detach().to(w.dtype).contiguous()
    return w, b


def _backward(ctx, dy):
    dy2, _ = as_rows(dy.to(torch.bfloat16))
    dx, dw = K.layernorm_bwd(dy2, ctx.saved, ctx.weight.detach().contiguous(), ctx.mean, ctx.rstd)
    db = dy2.float().sum(0).to(ctx.bias.dtype) if ctx.bias is not None else None
    return dx.reshape(dy.shape), dw, db


class EfficientMemoryLayerNormFunc(torch.autograd.Function):
    """apply(x, normalized_shape, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
    weight, bias, eps, iteration, static_value) -> (y, outlier, L, R, scale); backward: dx at slot 0, dw at 7, db at 8."""

    @staticmethod
    def forward(ctx, x, normalized_shape, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method,
                rank, weight, bias, eps, iteration, static_value):
        x = x.contiguous()
        x2, _ = as_rows(x)
        if x2.shape[-1] * x.element_size() > 65536:
            raise RuntimeError("This layer norm doesn't support feature dim >= 64KB.")
        if iteration < 2:
            outlier, L, R, scale = get_statistics(x, iteration, outlier_ratio, sub_outlier_ratio, sub_outlier_bit,
                                                  sub_outlier_quantize_method, rank)
        else:
            outlier, L, scale, R = static_value[0], static_value[1], static_value[2], static_value[3]
        if (sub_outlier_ratio > 0. and sub_outlier_bit != 16 and x.dim() == 3
                and K.layernorm_fwd_supported(x2.shape[-1], sub_outlier_bit)):
            w, b = _affine(weight, bias)
            y, mean, rstd, c = K.layernorm_fwd_compress_threshold(
                x2, w, b, eps, x.shape[-2], K.threshold_value(outlier), scale.contiguous(), sub_outlier_bit,
                L.contiguous() if rank > 0 else None, R.contiguous() if rank > 0 else None, budget=K.kept_budget(outlier))
        else:
            y, mean, rstd = _forward_stats(x2, weight, bias, eps)
            c, _ = compress_to_csr(x, outlier, scale, sub_outlier_bit, sub_outlier_ratio, L if rank > 0 else None,
                                   R if rank > 0 else None)
        ctx.saved, ctx.mean, ctx.rstd, ctx.weight, ctx.bias = c, mean, rstd, weight, bias
        ctx.mark_non_differentiable(outlier, L, R, scale)
        return y.reshape(x.shape), outlier, L, R, scale

    @staticmethod
    def backward(ctx, dy, grad_outlier, grad_L, grad_R, grad_scale):
        dx, dw, db = _backward(ctx, dy)
        return dx, None, None, None, None, None, None, dw, db, None, None, None


class _ChannelLayerNormFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, eps, plan, bits, group):
        x2, _ = as_rows(x)
        if K.layernorm_fwd_supported(x2.shape[-1], bits):
            w, b = _affine(weight, bias)
            y, mean, rstd, ctx.saved = K.layernorm_fwd_compress_channel(x2, w, b, eps, plan, bits, group)
        else:
            y, mean, rstd = _forward_stats(x2, weight, bias, eps)
            ctx.saved = K.compress_channel(x2, plan, bits, group)
        ctx.mean, ctx.rstd, ctx.weight, ctx.bias = mean, rstd, weight, bias
        return y.reshape(x.shape)

    @staticmethod
    def backward(ctx, dy):
        dx, dw, db = _backward(ctx, dy)
        return dx, dw, db, None, None, None, None


class EfficientMemoryLayerNorm(torch.nn.LayerNorm):
    def __init__(self, normalized_shape, eps=1e-05, elementwise_affine=True, bias=True, outlier_ratio: float = 0.01,
                 sub_outlier_ratio: float = 0.2, sub_outlier_bit: int = 8, sub_outlier_quantize_method: str = 'per-tensor',
                 rank: int = 16, *, mode: str = "ref", group_size: int = 128, scale_rule: str = "absmax"):
        super(EfficientMemoryLayerNorm, self).__init__(normalized_shape, eps, elementwise_affine, bias)
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

    def forward(self, x):
        if self.mode == "hyc":
            x2, _ = as_rows(x)
            plan = self.site.channel_plan(x2, self.iteration)
            y = _ChannelLayerNormFunc.apply(x, self.weight, self.bias, self.eps, plan, self.sub_outlier_bit, self.group_size)
            self.iteration += 1
            return y
        result, outlier, L, R, scale = EfficientMemoryLayerNormFunc.apply(
            x, self.normalized_shape, self.outlier_ratio, self.sub_outlier_ratio, self.sub_outlier_bit,
            self.sub_outlier_quantize_method, self.rank, self.weight, self.bias, self.eps, self.iteration,
            self.static_value)
        if self.iteration < 2:
            self.static_value = fold_statistics(self.static_value, self.iteration, outlier, L, scale, R)
        self.iteration += 1
        return result
