"""Calibration protocol shared by every operator module (reference: the block after Function.apply in each
module, e.g. operators/efficient_silu.py:86-111 or operators/efficient_rmsnorm.py:312-337).

Reference scheme ("ref" mode): `iteration` counts the calls; the first two calls compute fresh statistics
(threshold, L, scale, R), compress with them, and fold them into the running mean
`static = (iteration*static + fresh) / (iteration+1)`; from the third call on the stored values are used.
`static_value` keeps the reference's order [threshold, L, scale, R].  Like in the reference these are plain
Python attributes, not buffers.

Channel scheme ("hyc" mode): the state is the running per-channel abs-max (elementwise max over the first two
calls) and the outlier-channel plan selected from it; frozen from the third call on.
"""
import torch

from .. import kernels as K
from .compress_function import pad_cut_L

MODES = ("ref", "hyc")


def fold_statistics(static_value, iteration, outlier, L, scale, R):
    """one step of the running mean over the calibration calls; returns the new list"""
    fresh = [outlier, L, scale, R]
    out = list(static_value)
    for slot in range(4):
        new = fresh[slot]
        if out[slot] is None:
            out[slot] = new
        else:
            if slot == 1:
                new = pad_cut_L(new, out[slot])
            out[slot] = (iteration * out[slot] + new) / (iteration + 1)
    return out


class CompressionSite:
    """per-activation state: the reference's (iteration, static_value) pair plus the channel-mode plan"""

    def __init__(self, outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
                 mode="ref", group_size=128):
        if mode not in MODES:
            raise ValueError("mode must be 'ref' or 'hyc', got %r" % (mode,))
        self.outlier_ratio = outlier_ratio
        self.sub_outlier_ratio = sub_outlier_ratio
        self.sub_outlier_bit = sub_outlier_bit
        self.sub_outlier_quantize_method = sub_outlier_quantize_method
        self.rank = rank
        self.mode = mode
        self.group_size = group_size
        self.amax = None     # hyc mode: running channel abs-max (fp32 [H])
        self.plan = None     # hyc mode: ChannelPlan

    # -- channel mode ---------------------------------------------------------------------------------
    def channel_plan(self, x2d, iteration):
        """the plan to compress this call with; calibrates during the first two calls"""
        if iteration < 2 or self.plan is None:
            self.amax = K.channel_absmax(x2d, self.amax)
            k = K.num_outlier_channels(x2d.shape[-1], self.outlier_ratio)
            self.plan = K.select_channels(self.amax, k)
        return self.plan


def as_rows(x):
    """[..., H] -> contiguous [M, H] view plus the tokens-per-batch-element S the static scale is indexed by"""
    H = x.shape[-1]
    S = x.shape[-2] if x.dim() >= 2 else 1
    return x.contiguous().reshape(-1, H), S
