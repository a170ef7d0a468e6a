"""Attention matmuls with both operands saved compressed.  Reference: operators/efficient_gemm.py:13-330.

EfficientMemoryGEMM is `q @ kT` (x1 [B,nh,S,hd], x2 [B,nh,hd,S]; both saved as codes + outliers in the
[B,S,nh*hd] layout, x2 through its transpose, reference :39,:51).  EfficientMemoryGEMMWithSoftmax is `p @ v`
(x1 = attention probabilities [B,nh,S,S] saved as the entries above a threshold, x2 = v [B,nh,S,hd] saved as
codes + outliers, reference :222-223).  The two products themselves are plain batched library GEMMs; the
compress / decompress / sparsify work around them goes through the HIP kernels.
"""
import torch

from .. import kernels as K
from ._calibration import CompressionSite, fold_statistics, running_mean
from .compress_function import (compress_to_csr, get_statistics, get_statistics_softmax, head_to_hidden_shape,
                                hidden_to_head_shape)


def _calibrated(x, iteration, static, ratio, sub, bit, method, rank):
    if iteration < 2:
        return get_statistics(x, iteration, ratio, sub, bit, method, rank)     # (outlier, L, R, scale)
    return static[0], static[1], static[3], static[2]


def _restore_heads(c, shape, num_heads):
    """compressed [B*S, nh*hd] rows -> bf16 [B,nh,S,hd]"""
    return hidden_to_head_shape(K.decompress_threshold(c).reshape(shape), num_heads)


def _as_hidden_rows(x):
    """[B,nh,S,hd] -> contiguous [B*S, nh*hd] rows plus (B, S, nh)"""
    b, nh, s, hd = x.shape
    return head_to_hidden_shape(x).contiguous().reshape(b * s, nh * hd), (b, s, nh)


def _rows_to_heads(x2d, b, s, nh):
    return hidden_to_head_shape(x2d.reshape(b, s, -1), nh)


class EfficientMemoryGEMMFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1, x2, outlier_ratio_1, sub_outlier_ratio_1, sub_outlier_bit_1, sub_outlier_quantize_method_1,
                outlier_ratio_2, sub_outlier_ratio_2, sub_outlier_bit_2, sub_outlier_quantize_method_2, rank, iteration,
                static_value_1, static_value_2):
        result = x1 @ x2
        ctx.num_heads = x1.shape[1]
        x2t = x2.mT
        o1, L1, R1, s1 = _calibrated(x1, iteration, static_value_1, outlier_ratio_1, sub_outlier_ratio_1,
                                     sub_outlier_bit_1, sub_outlier_quantize_method_1, rank)
        o2, L2, R2, s2 = _calibrated(x2t, iteration, static_value_2, outlier_ratio_2, sub_outlier_ratio_2,
                                     sub_outlier_bit_2, sub_outlier_quantize_method_2, rank)
        c1, shape1 = compress_to_csr(x1, o1, s1, sub_outlier_bit_1, sub_outlier_ratio_1,
                                     L1 if rank > 0 else None, R1 if rank > 0 else None)
        c2, shape2 = compress_to_csr(x2t, o2, s2, sub_outlier_bit_2, sub_outlier_ratio_2,
                                     L2 if rank > 0 else None, R2 if rank > 0 else None)
        ctx.saved = (c1, shape1, c2, shape2)
        ctx.mark_non_differentiable(o1, o2, L1, R1, s1, L2, R2, s2)
        return result, o1, L1, R1, s1, o2, L2, R2, s2

    @staticmethod
    def backward(ctx, grad_output, *unused):
        c1, shape1, c2, shape2 = ctx.saved
        x1 = _restore_heads(c1, shape1, ctx.num_heads)
        x2t = _restore_heads(c2, shape2, ctx.num_heads)              # [B,nh,S,hd] = x2 transposed
        g = grad_output
        grad_input1 = g @ x2t.to(g.dtype)                            # g @ x2^T
        grad_input2 = x1.transpose(-2, -1).to(g.dtype) @ g
        return (grad_input1, grad_input2) + (None,) * 12


class _ChannelGEMMFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1, x2, plan1, plan2, bits1, bits2, group):
        r1, (b, s1, nh) = _as_hidden_rows(x1)
        r2, (_, s2, _) = _as_hidden_rows(x2.mT)
        ctx.saved = (K.compress_channel(r1, plan1, bits1, group), K.compress_channel(r2, plan2, bits2, group))
        ctx.geom = (b, s1, s2, nh)
        return x1 @ x2

    @staticmethod
    def backward(ctx, grad_output):
        b, s1, s2, nh = ctx.geom
        x1 = _rows_to_heads(K.decompress_channel(ctx.saved[0]), b, s1, nh)
        x2t = _rows_to_heads(K.decompress_channel(ctx.saved[1]), b, s2, nh)
        g = grad_output
        return g @ x2t.to(g.dtype), x1.transpose(-2, -1).to(g.dtype) @ g, None, None, None, None, None


class EfficientMemoryGEMM(torch.nn.Module):
    def __init__(self, outlier_ratio_1: float = 0.01, sub_outlier_ratio_1: float = 0.2, sub_outlier_bit_1: int = 8,
                 sub_outlier_quantize_method_1: str = 'per-tensor', outlier_ratio_2: float = 0.01,
                 sub_outlier_ratio_2: float = 0.2, sub_outlier_bit_2: int = 8,
                 sub_outlier_quantize_method_2: str = 'per-tensor', rank: int = 16, *, mode: str = "ref",
                 group_size: int = 128, scale_rule: str = "absmax"):
        super().__init__()
        self.outlier_ratio_1, self.sub_outlier_ratio_1 = outlier_ratio_1, sub_outlier_ratio_1
        self.sub_outlier_bit_1, self.sub_outlier_quantize_method_1 = sub_outlier_bit_1, sub_outlier_quantize_method_1
        self.outlier_ratio_2, self.sub_outlier_ratio_2 = outlier_ratio_2, sub_outlier_ratio_2
        self.sub_outlier_bit_2, self.sub_outlier_quantize_method_2 = sub_outlier_bit_2, sub_outlier_quantize_method_2
        self.rank = rank
        self.mode = mode
        self.group_size = group_size
        self.site_1 = CompressionSite(outlier_ratio_1, sub_outlier_ratio_1, sub_outlier_bit_1,
                                      sub_outlier_quantize_method_1, rank, mode, group_size, scale_rule)
        self.site_2 = CompressionSite(outlier_ratio_2, sub_outlier_ratio_2, sub_outlier_bit_2,
                                      sub_outlier_quantize_method_2, rank, mode, group_size, scale_rule)
        self.iteration = 0
        self.static_value_1 = [None, None, None, None]
        self.static_value_2 = [None, None, None, None]

    def forward(self, x1, x2):
        if self.mode == "hyc":
            r1, _ = _as_hidden_rows(x1)
            r2, _ = _as_hidden_rows(x2.mT)
            p1 = self.site_1.channel_plan(r1, self.iteration)
            p2 = self.site_2.channel_plan(r2, self.iteration)
            result = _ChannelGEMMFunc.apply(x1, x2, p1, p2, self.sub_outlier_bit_1, self.sub_outlier_bit_2,
                                            self.group_size)
            self.iteration += 1
            return result
        result, o1, L1, R1, s1, o2, L2, R2, s2 = EfficientMemoryGEMMFunc.apply(
            x1, x2, self.outlier_ratio_1, self.sub_outlier_ratio_1, self.sub_outlier_bit_1,
            self.sub_outlier_quantize_method_1, self.outlier_ratio_2, self.sub_outlier_ratio_2, self.sub_outlier_bit_2,
            self.sub_outlier_quantize_method_2, self.rank, self.iteration, self.static_value_1, self.static_value_2)
        if self.iteration < 2:
            self.static_value_1 = fold_statistics(self.static_value_1, self.iteration, o1, L1, s1, R1)
            self.static_value_2 = fold_statistics(self.static_value_2, self.iteration, o2, L2, s2, R2)
        self.iteration += 1
        return result


class EfficientMemoryGEMMWithSoftmaxFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1, x2, outlier_ratio_1, outlier_ratio_2, sub_outlier_ratio_2, sub_outlier_bit_2,
                sub_outlier_quantize_method_2, rank, iteration, static_value_1, static_value_2):
        result = x1 @ x2
        ctx.num_heads = x1.shape[1]
        o1 = get_statistics_softmax(x1, iteration, outlier_ratio_1) if iteration < 2 else static_value_1
        o2, L2, R2, s2 = _calibrated(x2, iteration, static_value_2, outlier_ratio_2, sub_outlier_ratio_2,
                                     sub_outlier_bit_2, sub_outlier_quantize_method_2, rank)
        ctx.sparse = K.softmax_sparsify(x1.contiguous(), K.threshold_value(o1), budget=K.kept_budget(o1))
        c2, shape2 = compress_to_csr(x2, o2, s2, sub_outlier_bit_2, sub_outlier_ratio_2,
                                     L2 if rank > 0 else None, R2 if rank > 0 else None)
        ctx.saved = (c2, shape2)
        ctx.mark_non_differentiable(o1, o2, L2, R2, s2)
        return result, o1, o2, L2, R2, s2

    @staticmethod
    def backward(ctx, grad_output, *unused):
        c2, shape2 = ctx.saved
        x1 = K.softmax_dense(ctx.sparse)
        x2 = _restore_heads(c2, shape2, ctx.num_heads)
        g = grad_output
        grad_input1 = g @ x2.transpose(-2, -1).to(g.dtype)
        grad_input2 = x1.transpose(-2, -1).to(g.dtype) @ g
        return (grad_input1, grad_input2) + (None,) * 9


class _ChannelGEMMWithSoftmaxFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1, x2, threshold, plan2, bits2, group):
        r2, (b, s2, nh) = _as_hidden_rows(x2)
        ctx.sparse = K.softmax_sparsify(x1.contiguous(), K.threshold_value(threshold), budget=K.kept_budget(threshold))
        ctx.saved = K.compress_channel(r2, plan2, bits2, group)
        ctx.geom = (b, s2, nh)
        return x1 @ x2

    @staticmethod
    def backward(ctx, grad_output):
        b, s2, nh = ctx.geom
        x1 = K.softmax_dense(ctx.sparse)
        x2 = _rows_to_heads(K.decompress_channel(ctx.saved), b, s2, nh)
        g = grad_output
        return g @ x2.transpose(-2, -1).to(g.dtype), x1.transpose(-2, -1).to(g.dtype) @ g, None, None, None, None


class EfficientMemoryGEMMWithSoftmax(torch.nn.Module):
    def __init__(self, outlier_ratio_1: float = 0.01, outlier_ratio_2: float = 0.01, sub_outlier_ratio_2: float = 0.2,
                 sub_outlier_bit_2: int = 8, sub_outlier_quantize_method_2: str = 'per-tensor', rank: int = 16, *,
                 mode: str = "ref", group_size: int = 128, scale_rule: str = "absmax"):
        super().__init__()
        self.outlier_ratio_1 = outlier_ratio_1
        self.outlier_ratio_2, self.sub_outlier_ratio_2 = outlier_ratio_2, sub_outlier_ratio_2
        self.sub_outlier_bit_2, self.sub_outlier_quantize_method_2 = sub_outlier_bit_2, sub_outlier_quantize_method_2
        self.rank = rank
        self.mode = mode
        self.group_size = group_size
        self.site_2 = CompressionSite(outlier_ratio_2, sub_outlier_ratio_2, sub_outlier_bit_2,
                                      sub_outlier_quantize_method_2, rank, mode, group_size, scale_rule)
        self.iteration = 0
        self.static_value_1 = None
        self.static_value_2 = [None, None, None, None]

    def forward(self, x1, x2):
        if self.mode == "hyc":
            # the probabilities keep the reference's threshold rule; only v uses the channel scheme
            if self.iteration < 2:
                o1 = get_statistics_softmax(x1, self.iteration, self.outlier_ratio_1)
                self.static_value_1 = running_mean(self.static_value_1, o1, self.iteration)
            else:
                o1 = self.static_value_1
            r2, _ = _as_hidden_rows(x2)
            p2 = self.site_2.channel_plan(r2, self.iteration)
            result = _ChannelGEMMWithSoftmaxFunc.apply(x1, x2, o1, p2, self.sub_outlier_bit_2, self.group_size)
            self.iteration += 1
            return result
        result, o1, o2, L2, R2, s2 = EfficientMemoryGEMMWithSoftmaxFunc.apply(
            x1, x2, self.outlier_ratio_1, self.outlier_ratio_2, self.sub_outlier_ratio_2, self.sub_outlier_bit_2,
            self.sub_outlier_quantize_method_2, self.rank, self.iteration, self.static_value_1, self.static_value_2)
        if self.iteration < 2:
            self.static_value_1 = running_mean(self.static_value_1, o1, self.iteration)
            self.static_value_2 = fold_statistics(self.static_value_2, self.iteration, o2, L2, s2, R2)
        self.iteration += 1
        return result
