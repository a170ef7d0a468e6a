"""Elementwise product with both operands saved compressed.  Reference: operators/efficient_hadamard.py:9-183."""
import torch

from .. import kernels as K
from ._calibration import CompressionSite, as_rows, fold_statistics
from .compress_function import compress_to_csr, get_statistics


class EfficientMemoryHadamardFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1, x2, outlier_ratio_1, sub_outlier_ratio_1, sub_outlier_bit_1, sub_outlier_quantize_method_1,
                outlier_ratio_2, sub_outlier_ratio_2, sub_outlier_bit_2, sub_outlier_quantize_method_2, rank, iteration,
                static_value_1, static_value_2):
        result = x1 * x2
        stats = []
        for x, ratio, sub, bit, method, static in (
                (x1, outlier_ratio_1, sub_outlier_ratio_1, sub_outlier_bit_1, sub_outlier_quantize_method_1, static_value_1),
                (x2, outlier_ratio_2, sub_outlier_ratio_2, sub_outlier_bit_2, sub_outlier_quantize_method_2, static_value_2)):
            if iteration < 2:
                outlier, L, R, scale = get_statistics(x, iteration, ratio, sub, bit, method, rank)
            else:
                outlier, L, scale, R = static[0], static[1], static[2], static[3]
            c, shape = compress_to_csr(x, outlier, scale, bit, sub, L if rank > 0 else None, R if rank > 0 else None)
            stats.append((outlier, L, R, scale, c, shape))
        ctx.saved = (stats[0][4], stats[1][4])
        ctx.shape = stats[0][5]
        o1, L1, R1, s1 = stats[0][:4]
        o2, L2, R2, s2 = stats[1][:4]
        ctx.mark_non_differentiable(o1, o2, L1, R1, s1, L2, R2, s2)
        return result, o1, L1, R1, s1, o2, L2, R2, s2

    @staticmethod
    def backward(ctx, grad_output, *unused):
        g2, _ = as_rows(grad_output.to(torch.bfloat16))
        d1, d2 = K.hadamard_bwd(g2, ctx.saved[0], ctx.saved[1])
        return (d1.reshape(grad_output.shape), d2.reshape(grad_output.shape)) + (None,) * 12


class _ChannelHadamardFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1, x2, plan1, plan2, bits1, bits2, group):
        a, _ = as_rows(x1)
        b, _ = as_rows(x2)
        if a.shape == b.shape and K.hadamard_fwd_compress_supported(a.shape[-1], bits1, group, bits2, group):
            y, c1, c2 = K.hadamard_fwd_compress(a, b, plan1, plan2, bits1, group)      # each operand read once
            ctx.saved = (c1, c2)
            return y.view(x1.shape)
        ctx.saved = (K.compress_channel(a, plan1, bits1, group), K.compress_channel(b, plan2, bits2, group))
        return x1 * x2

    @staticmethod
    def backward(ctx, grad_output):
        g2, _ = as_rows(grad_output.to(torch.bfloat16))
        d1, d2 = K.hadamard_bwd(g2, ctx.saved[0], ctx.saved[1])
        return d1.reshape(grad_output.shape), d2.reshape(grad_output.shape), None, None, None, None, None


class EfficientMemoryHadamard(torch.nn.Module):
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
            a, _ = as_rows(x1)
            b, _ = as_rows(x2)
            p1 = self.site_1.channel_plan(a, self.iteration)
            p2 = self.site_2.channel_plan(b, self.iteration)
            result = _ChannelHadamardFunc.apply(x1, x2, p1, p2, self.sub_outlier_bit_1, self.sub_outlier_bit_2, self.group_size)
            self.iteration += 1
            return result
        result, o1, L1, R1, s1, o2, L2, R2, s2 = EfficientMemoryHadamardFunc.apply(
            x1, x2, self.outlier_ratio_1, self.sub_outlier_ratio_1, self.sub_outlier_bit_1,
            self.sub_outlier_quantize_method_1, self.outlier_ratio_2, self.sub_outlier_ratio_2, self.sub_outlier_bit_2,
            self.sub_outlier_quantize_method_2, self.rank, self.iteration, self.static_value_1, self.static_value_2)
        if self.iteration < 2:
            self.static_value_1 = fold_statistics(self.static_value_1, self.iteration, o1, L1, s1, R1)
            self.static_value_2 = fold_statistics(self.static_value_2, self.iteration, o2, L2, s2, R2)
        self.iteration += 1
        return result


def _row_view(t):
    """[..., H] -> [M, H] without a copy when the rows are evenly spaced (e.g. a column slice of a fused projection)"""
    H = t.shape[-1]
    if t.stride(-1) != 1:
        t = t.contiguous()
    try:
        return t.view(-1, H)
    except RuntimeError:
        return t.reshape(-1, H)


class _ChannelGatedActFunc(torch.autograd.Function):
    """h = act(gate) * up with the three activations EfficientMemorySiLU/GELU and EfficientMemoryHadamard would save
    (gate; act(gate) and up), and one backward pass over them."""

    @staticmethod
    def forward(ctx, gate, up, act, sites, iteration, bits, group):
        ctx.act = act
        calibrated = iteration >= 2 and all(site.plan is not None for site in sites)
        if calibrated and K.gated_act_fwd_supported(gate.shape[-1], bits, group):
            # steady state: one pass over gate and up writes the product and the three compressed activations;
            # act(gate) is never held in memory
            h, c_act, c_up, c_gate = K.gated_act_fwd(act, _row_view(gate), _row_view(up), sites[0].plan, sites[1].plan,
                                                     sites[2].plan, bits, group)
            ctx.saved = (c_act, c_up, c_gate)
            return h.view(gate.shape)
        # calibration calls need act(gate) as a tensor (its channel maxima choose the outlier channels)
        a = torch.nn.functional.silu(gate) if act == "silu" else torch.nn.functional.gelu(gate)
        rows = [_row_view(t) for t in (a, up, gate)]
        ctx.saved = tuple(K.compress_channel(r, site.channel_plan(r, iteration), bits, group)
                          for r, site in zip(rows, sites))
        return a * up

    @staticmethod
    def backward(ctx, grad_output):
        g2, _ = as_rows(grad_output.to(torch.bfloat16))
        d_gate, d_up = K.gated_act_bwd(ctx.act, g2, *ctx.saved)
        return d_gate.reshape(grad_output.shape), d_up.reshape(grad_output.shape), None, None, None, None, None


class EfficientMemoryGatedAct(torch.nn.Module):
    """SwiGLU / GeGLU product `act(gate) * up` as one module (channel scheme only).  The reference composes
    EfficientMemorySiLU (efficient_silu.py:56-113) and EfficientMemoryHadamard (efficient_hadamard.py:86-183); this
    module saves the same three compressed activations and gives bit-identical gradients, but its backward reads the
    incoming gradient once and never writes the gradient of act(gate) to memory."""

    def __init__(self, act: str = "silu", outlier_ratio: float = 0.01, sub_outlier_ratio: float = 1.0,
                 sub_outlier_bit: int = 4, sub_outlier_quantize_method: str = 'per-token', rank: int = 0, *,
                 group_size: int = 128, scale_rule: str = "absmax"):
        super().__init__()
        if act not in ("silu", "gelu"):
            raise ValueError("act must be 'silu' or 'gelu'")
        self.act, self.sub_outlier_bit, self.group_size = act, sub_outlier_bit, group_size
        mk = lambda: CompressionSite(outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method,
                                     rank, "hyc", group_size, scale_rule)
        self.site_act, self.site_up, self.site_gate = mk(), mk(), mk()
        self.iteration = 0

    def forward(self, gate, up):
        out = _ChannelGatedActFunc.apply(gate, up, self.act, (self.site_act, self.site_up, self.site_gate), self.iteration,
                                         self.sub_outlier_bit, self.group_size)
        self.iteration += 1
        return out
