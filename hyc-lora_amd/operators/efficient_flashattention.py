"""Fused attention over packed variable-length sequences, with q, k, v and the attention output saved compressed and
the backward kernel run on the restored tensors.  Reference: operators/efficient_flashattention.py:10-302.

The reference drives flash_attn's `_flash_attn_varlen_forward / _backward`; that package is not part of this
environment, so the fused kernels are the framework's own (`aten::_scaled_dot_product_flash_attention` and its
backward), called once for the whole batch when every sequence has the same length and once per sequence otherwise.
What the reference's operator is about is unchanged: no [S, S] tensor exists, the forward keeps four compressed
activations plus one fp32 log-sum-exp per (head, token), and the backward kernel receives decompressed q, k, v, out
(its row term sum(dO * O) therefore comes from the restored output, :97-134).
"""
import torch

from .. import kernels as K
from ._calibration import CompressionSite, fold_statistics
from .compress_function import compress_to_csr, get_statistics

_CALIBRATION_CALLS = 5          # the reference averages the statistics of the first five calls here (:66, :197)


def _check_unsupported(window_size, alibi_slopes):
    if tuple(window_size) != (-1, -1):
        raise NotImplementedError("sliding-window attention is outside the accelerated path")
    if alibi_slopes is not None:
        raise NotImplementedError("ALiBi slopes are outside the accelerated path")


def _sequence_bounds(cu_seqlens, total):
    """host list of the cumulative sequence lengths (one read-back per call; max_seqlen is a host integer in the
    reference's signature already)"""
    bounds = [int(v) for v in cu_seqlens.tolist()]
    if len(bounds) < 2 or bounds[0] != 0 or bounds[-1] != total or any(b <= a for a, b in zip(bounds, bounds[1:])):
        raise ValueError("cu_seqlens must rise from 0 to the number of packed tokens (%d), got %s" % (total, bounds))
    return bounds


def _segments(bounds):
    """[(first token, sequences, length)]: the whole batch as one segment when the lengths agree"""
    lens = [b - a for a, b in zip(bounds, bounds[1:])]
    if all(n == lens[0] for n in lens):
        return [(0, len(lens), lens[0])]
    return [(a, 1, n) for a, n in zip(bounds, lens)]


def _heads_view(t, first, count, length):
    """tokens [first, first + count*length) of t [total, nh, hd] (any token pitch) as [count, nh, length, hd]"""
    nh, hd = t.shape[1], t.shape[2]
    return t[first:first + count * length].unflatten(0, (count, length)).transpose(1, 2)


def _attention_forward(q, k, v, bounds, dropout_p, scale, causal):
    """q, k, v [total, nh, hd] -> (out [total, nh, hd] contiguous, per-segment (log-sum-exp, rng seed, rng offset))"""
    total, nh, hd = q.shape
    out = torch.empty((total, nh, hd), dtype=q.dtype, device=q.device)
    state = []
    for first, count, length in _segments(bounds):
        o, lse, _, _, _, _, seed, offset, _ = torch.ops.aten._scaled_dot_product_flash_attention(
            _heads_view(q, first, count, length), _heads_view(k, first, count, length),
            _heads_view(v, first, count, length), dropout_p, causal, False, scale=scale)
        _heads_view(out, first, count, length).copy_(o)
        state.append((lse, seed, offset))
    return out, state


def _attention_backward(dout, q, k, v, out, state, bounds, dropout_p, scale, causal):
    """-> dqkv [total, 3, nh, hd] from restored q, k, v, out [total, nh, hd]"""
    total, nh, hd = q.shape
    dqkv = torch.empty((total, 3, nh, hd), dtype=q.dtype, device=q.device)
    for (first, count, length), (lse, seed, offset) in zip(_segments(bounds), state):
        view = lambda t: _heads_view(t, first, count, length)
        grads = torch.ops.aten._scaled_dot_product_flash_attention_backward(
            view(dout), view(q), view(k), view(v), view(out), lse, None, None, length, length, dropout_p, causal,
            seed, offset, scale=scale)
        for slot, gslot in enumerate(grads):
            view(dqkv[:, slot]).copy_(gslot)
    return dqkv


class EfficientFlashAttnVarlenQKVPackedFunc(torch.autograd.Function):
    """apply(qkv [total, 3, nh, hd], cu_seqlens, max_seqlen, dropout_p, softmax_scale, causal, window_size,
    alibi_slopes, deterministic, return_softmax, outlier_ratio, sub_outlier_ratio, sub_outlier_bit,
    sub_outlier_quantize_method, rank, iteration, q_static_value, k_static_value, v_static_value, o_static_value)
    -> (out [total, nh, hd], q/k/v/o outlier, q/k/v/o scale, q_L, q_R, k_L, k_R, v_L, v_R, o_L, o_R), the order of
    the reference (:94)."""

    @staticmethod
    def forward(ctx, qkv, cu_seqlens, max_seqlen, dropout_p, softmax_scale, causal, window_size, alibi_slopes,
                deterministic, return_softmax, outlier_ratio, sub_outlier_ratio, sub_outlier_bit,
                sub_outlier_quantize_method, rank, iteration, q_static_value, k_static_value, v_static_value,
                o_static_value):
        _check_unsupported(window_size, alibi_slopes)
        total, three, nh, hd = qkv.shape
        if three != 3:
            raise ValueError("qkv must be [tokens, 3, heads, head_dim]")
        scale = hd ** (-0.5) if softmax_scale is None else softmax_scale
        bounds = _sequence_bounds(cu_seqlens, total)
        out, state = _attention_forward(qkv[:, 0], qkv[:, 1], qkv[:, 2], bounds, dropout_p, scale, causal)
        # the reference compresses [1, nh, total, hd] tensors, which its helpers turn into [1, total, nh*hd] first
        # (compress_function.py:138-141): the same rows, taken here without the two permutations
        rows = [qkv[:, 0].reshape(1, total, nh * hd), qkv[:, 1].reshape(1, total, nh * hd),
                qkv[:, 2].reshape(1, total, nh * hd), out.view(1, total, nh * hd)]
        stats, saved = [], []
        for x, static in zip(rows, (q_static_value, k_static_value, v_static_value, o_static_value)):
            if iteration < _CALIBRATION_CALLS:
                outlier, L, R, scale_x = get_statistics(x, iteration, outlier_ratio, sub_outlier_ratio, sub_outlier_bit,
                                                        sub_outlier_quantize_method, rank)
            else:
                outlier, L, scale_x, R = static[0], static[1], static[2], static[3]
            c, _ = compress_to_csr(x, outlier, scale_x, sub_outlier_bit, sub_outlier_ratio,
                                   L if rank > 0 else None, R if rank > 0 else None)
            stats.append((outlier, L, R, scale_x))
            saved.append(c)
        ctx.saved, ctx.state, ctx.bounds = saved, state, bounds
        ctx.dropout_p, ctx.scale, ctx.causal, ctx.geom = dropout_p, scale, causal, (total, nh, hd)
        (qo, qL, qR, qs), (ko, kL, kR, ks), (vo, vL, vR, vs), (oo, oL, oR, os_) = stats
        ctx.mark_non_differentiable(qo, ko, vo, oo, qs, ks, vs, os_, qL, qR, kL, kR, vL, vR, oL, oR)
        return out, qo, ko, vo, oo, qs, ks, vs, os_, qL, qR, kL, kR, vL, vR, oL, oR

    @staticmethod
    def backward(ctx, dout, *args):
        total, nh, hd = ctx.geom
        q, k, v, out = (K.decompress_threshold(c).view(total, nh, hd) for c in ctx.saved)
        ctx.saved = None
        dqkv = _attention_backward(dout.to(q.dtype).contiguous(), q, k, v, out, ctx.state, ctx.bounds, ctx.dropout_p,
                                   ctx.scale, ctx.causal)
        return (dqkv,) + (None,) * 19


class _ChannelFlashAttnFunc(torch.autograd.Function):
    """channel-scheme twin: q, k, v are read as column slices of the packed tensor (row pitch 3*nh*hd), no copies"""

    @staticmethod
    def forward(ctx, qkv, bounds, dropout_p, scale, causal, sites, iteration, bits, group):
        total, _, nh, hd = qkv.shape
        out, state = _attention_forward(qkv[:, 0], qkv[:, 1], qkv[:, 2], bounds, dropout_p, scale, causal)
        packed = qkv.view(total, 3 * nh * hd)
        rows = [packed[:, i * nh * hd:(i + 1) * nh * hd] for i in range(3)] + [out.view(total, nh * hd)]
        ctx.saved = [K.compress_channel(r, site.channel_plan(r, iteration), bits, group) for r, site in zip(rows, sites)]
        ctx.state, ctx.bounds = state, bounds
        ctx.dropout_p, ctx.scale, ctx.causal, ctx.geom = dropout_p, scale, causal, (total, nh, hd)
        return out

    @staticmethod
    def backward(ctx, dout):
        total, nh, hd = ctx.geom
        q, k, v, out = (K.decompress_channel(c).view(total, nh, hd) for c in ctx.saved)
        ctx.saved = None
        dqkv = _attention_backward(dout.to(q.dtype).contiguous(), q, k, v, out, ctx.state, ctx.bounds, ctx.dropout_p,
                                   ctx.scale, ctx.causal)
        return (dqkv,) + (None,) * 8


class EfficientFlashAttnVarlenQKVPacked(torch.nn.Module):
    """forward(qkv, cu_seqlens, max_seqlen, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
    alibi_slopes=None, deterministic=False, return_attn_probs=False) -> out [total, nh, hd].  (The reference's
    forward ends without a return statement, :302; the attention output is what its Function computes.)"""

    def __init__(self, outlier_ratio: float = 0.01, sub_outlier_ratio: float = 0.2, sub_outlier_bit: int = 8,
                 sub_outlier_quantize_method: str = 'per-tensor', rank: int = 16, *, mode: str = "ref",
                 group_size: int = 128, scale_rule: str = "absmax"):
        super(EfficientFlashAttnVarlenQKVPacked, self).__init__()
        self.outlier_ratio = outlier_ratio
        self.sub_outlier_ratio = sub_outlier_ratio
        self.sub_outlier_bit = sub_outlier_bit
        self.sub_outlier_quantize_method = sub_outlier_quantize_method
        self.rank = rank
        self.mode = mode
        self.group_size = group_size
        mk = lambda: CompressionSite(outlier_ratio, sub_outlier_ratio, sub_outlier_bit, sub_outlier_quantize_method, rank,
                                     mode, group_size, scale_rule)
        self.site_q, self.site_k, self.site_v, self.site_o = mk(), mk(), mk(), mk()
        self.iteration = 0
        self.q_static_value = [None, None, None, None]
        self.k_static_value = [None, None, None, None]
        self.v_static_value = [None, None, None, None]
        self.o_static_value = [None, None, None, None]

    def forward(self, qkv, cu_seqlens, max_seqlen, dropout_p=0.0, softmax_scale=None, causal=False, window_size=(-1, -1),
                alibi_slopes=None, deterministic=False, return_attn_probs=False):
        if self.mode == "hyc":
            _check_unsupported(window_size, alibi_slopes)
            if qkv.dim() != 4 or qkv.shape[1] != 3 or not qkv.is_contiguous():
                raise ValueError("qkv must be a contiguous [tokens, 3, heads, head_dim] tensor")
            scale = qkv.shape[-1] ** (-0.5) if softmax_scale is None else softmax_scale
            out = _ChannelFlashAttnFunc.apply(qkv, _sequence_bounds(cu_seqlens, qkv.shape[0]), dropout_p, scale, causal,
                                              (self.site_q, self.site_k, self.site_v, self.site_o), self.iteration,
                                              self.sub_outlier_bit, self.group_size)
            self.iteration += 1
            return out
        (out, qo, ko, vo, oo, qs, ks, vs, os_, qL, qR, kL, kR, vL, vR, oL, oR) = EfficientFlashAttnVarlenQKVPackedFunc.apply(
            qkv, cu_seqlens, max_seqlen, dropout_p, softmax_scale, causal, window_size, alibi_slopes, deterministic,
            return_attn_probs, self.outlier_ratio, self.sub_outlier_ratio, self.sub_outlier_bit,
            self.sub_outlier_quantize_method, self.rank, self.iteration, self.q_static_value, self.k_static_value,
            self.v_static_value, self.o_static_value)
        if self.iteration < _CALIBRATION_CALLS:
            self.q_static_value = fold_statistics(self.q_static_value, self.iteration, qo, qL, qs, qR)
            self.k_static_value = fold_statistics(self.k_static_value, self.iteration, ko, kL, ks, kR)
            self.v_static_value = fold_statistics(self.v_static_value, self.iteration, vo, vL, vs, vR)
            self.o_static_value = fold_statistics(self.o_static_value, self.iteration, oo, oL, os_, oR)
        self.iteration += 1
        return out
