"""One LLaMA-shaped decoder layer with a 4-bit NF4 frozen base, LoRA on all seven projections and every saved
activation compressed: the harness for the full-layer configuration (peak activation memory and step time).

What the reference assembles by swapping modules inside models/modeling_llama.py (attention :382-484, MLP
:263-295) with peft LoRA around a bitsandbytes 4-bit base (bitsandbytes_fix/_function.py:509-540) is built here
directly from this package's operators, with the savings a hand-assembled layer allows:

* q/k/v (and gate/up) LoRA-A inputs are the same tensor: it is compressed once, not once per projection;
* the attention probabilities are kept once (the reference keeps them in the softmax module and again in the
  p @ v wrapper, efficient_gemm.py:222);
* the frozen base saves nothing (as in the reference): W is dequantised again in the backward.

Composite of one LoRA projection (peft `Linear.forward` around the swapped modules):
    y  = x @ W^T + s * (x @ A^T) @ B^T          h = x @ A^T is kept exactly ([M, r])
    dX = dY @ W + (s * dY @ B) @ A
    dB = s * dY^T @ h
    dA = (s * dY @ B)^T @ x_hat                 the only consumer of the compressed x (efficient_linear.py:56-67)
"""
import math
from dataclasses import dataclass

import torch

from . import kernels as K
from .operators._calibration import CompressionSite, running_mean
from .operators.compress_function import get_statistics_softmax
from .operators.efficient_hadamard import EfficientMemoryGatedAct
from .operators.efficient_rmsnorm import EfficientMemoryRMSNorm

BF16 = torch.bfloat16


@dataclass
class LayerConfig:
    hidden: int = 4096
    heads: int = 32
    head_dim: int = 128
    intermediate: int = 11008
    rope_theta: float = 10000.0
    rms_eps: float = 1e-5
    lora_r: int = 16
    lora_alpha: float = 32.0
    outlier_ratio: float = 0.01      # fraction of channels kept in bf16 at every compressed site
    softmax_ratio: float = 0.01      # fraction of attention probabilities kept
    linear_bits: int = 2             # LoRA-A inputs
    linear_group: int = 64
    act_bits: int = 4                # norm inputs, q / k / v, gate / act(gate) / up
    act_group: int = 128
    scale_rule: str = "absmax"       # how a (token, group) scale is formed, see kernels.ChannelPlan
    compress: bool = True            # False: the same functions keep their activations in bf16 (formula check)
    attention: str = "eager"         # "eager": scores, softmax, p @ v with the kept probabilities (the path the
                                     # reference wires into its models); "flash": the library's fused attention with
                                     # q, k, v and the output saved as codes (operators/efficient_flashattention.py)
    attn_group_bytes: int = 128 << 20  # attention is walked in groups of [S, S] score matrices of at most this size


# ---- frozen base + LoRA -----------------------------------------------------------------------------------
class LoRAProjections(torch.nn.Module):
    """n projections of one input: frozen NF4 base W_i [out_i, in] plus trainable A_i [r, in], B_i [out_i, r]"""

    def __init__(self, in_features, out_features, cfg: LayerConfig, device):
        super().__init__()
        gen = torch.Generator(device="cpu").manual_seed(in_features * 31 + sum(out_features))
        self.in_features, self.out_features = in_features, list(out_features)
        self.scaling = cfg.lora_alpha / cfg.lora_r
        self.cfg = cfg
        self.lora_A = torch.nn.ParameterList()
        self.lora_B = torch.nn.ParameterList()
        weights = []
        for out in self.out_features:
            weights.append((0.02 * torch.randn(out, in_features, generator=gen)).to(BF16).to(device))
            a = torch.empty(cfg.lora_r, in_features)
            torch.nn.init.kaiming_uniform_(a, a=math.sqrt(5), generator=gen)
            self.lora_A.append(torch.nn.Parameter(a.to(BF16).to(device)))
            # peft starts B at zero; a small random B keeps every gradient of the harness non-trivial
            self.lora_B.append(torch.nn.Parameter((0.02 * torch.randn(out, cfg.lora_r, generator=gen)).to(BF16).to(device)))
        # the frozen weights of the group live as one [sum(out), in] NF4 matrix: one dequantisation and one base GEMM
        # per forward (a three times wider GEMM runs 15-25 % faster than three); base[i] are views of projection i
        self.base_all = K.nf4_quantize(torch.cat(weights, dim=0))
        del weights
        self.base, row = [], 0
        for out in self.out_features:
            lo, hi = row * in_features, (row + out) * in_features
            self.base.append(K.NF4Weight(self.base_all.packed[lo // 2:hi // 2], self.base_all.absmax[lo // 64:hi // 64],
                                         (out, in_features)))
            row += out
        self.site = CompressionSite(cfg.outlier_ratio, 1.0, cfg.linear_bits, "per-token", 0, "hyc", cfg.linear_group,
                                    cfg.scale_rule)
        self.iteration = 0
        self.record = None
        self._fused_choice = {}

    def fuse_base_gemm(self, x2, w_all):
        """whether the group's base GEMM runs faster as one wide GEMM or as one per projection: measured once per
        token count (the library's kernel selection favours either, depending on the shape: at 2048 tokens the
        fused gate/up GEMM is 30 % slower than two, at 4096 tokens 20 % faster)"""
        M = x2.shape[0]
        if len(self.out_features) == 1:
            return True
        if M not in self._fused_choice:
            scratch = torch.empty((M, sum(self.out_features)), dtype=BF16, device=x2.device)
            times = []
            for fused in (True, False):
                _base_gemm(scratch, x2, w_all, self.out_features, fused)                      # warm-up
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(3):
                    _base_gemm(scratch, x2, w_all, self.out_features, fused)
                e1.record()
                e1.synchronize()
                times.append(e0.elapsed_time(e1))
            self._fused_choice[M] = times[0] <= times[1]
        return self._fused_choice[M]

    def forward(self, x):
        x2 = x.reshape(-1, self.in_features)
        plan = self.site.channel_plan(x2, self.iteration) if self.cfg.compress else None
        self.iteration += 1
        n = len(self.out_features)
        outs = _LoRAProjectionsFunc.apply(x, self, plan, *self.lora_A, *self.lora_B)
        return outs if n > 1 else outs[0]


def _base_gemm(y_all, x2, w_all, out_features, fused):
    """y_all += x2 @ w_all^T, as one GEMM or as one GEMM per projection writing its column slice of y_all"""
    if fused or len(out_features) == 1:
        y_all.addmm_(x2, w_all.t())
        return
    row = 0
    for out in out_features:
        y_all[:, row:row + out].addmm_(x2, w_all[row:row + out].t())
        row += out


class _LoRAProjectionsFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, mod, plan, *ab):
        n = len(mod.out_features)
        A, B = ab[:n], ab[n:]
        r = A[0].shape[0]
        x2 = x.reshape(-1, mod.in_features)
        if not x2.is_contiguous():
            x2 = x2.contiguous()
        s = mod.scaling
        zero = x2.new_zeros(1)                                   # ignored (beta = 0), only has to broadcast
        total = sum(mod.out_features)
        # h = x A^T for every projection of the group at once; the rank-r terms s * h_i B_i^T as one thin GEMM with
        # the B_i on a block diagonal; then the base GEMM accumulates onto that in its epilogue (the other order
        # costs a separate read-modify-write pass over y)
        h_all = x2 @ (A[0] if n == 1 else torch.cat(list(A), dim=0)).t()                      # [M, n*r]
        if n == 1:
            b_all = B[0]
        else:
            b_all = x2.new_zeros((total, n * r))
            row = 0
            for i, out in enumerate(mod.out_features):
                b_all[row:row + out, i * r:(i + 1) * r] = B[i]
                row += out
        y_all = torch.addmm(zero, h_all, b_all.t(), beta=0.0, alpha=s)                         # [M, sum(out)]
        w_all = K.nf4_dequantize(mod.base_all)
        _base_gemm(y_all, x2, w_all, mod.out_features, mod.fuse_base_gemm(x2, w_all))
        del w_all, b_all
        outs, row = [], 0
        for out in mod.out_features:                            # column slices: no copies, consumers take the pitch
            outs.append(y_all[:, row:row + out].unflatten(0, x.shape[:-1]))
            row += out
        cfg = mod.cfg
        ctx.saved_x = K.compress_channel(x2, plan, cfg.linear_bits, cfg.linear_group) if cfg.compress else x2
        if mod.record is not None:
            mod.record["x"], mod.record["saved"] = x2.detach().clone(), ctx.saved_x
        ctx.mod, ctx.h_all = mod, h_all
        ctx.save_for_backward(*ab)
        return tuple(outs)

    @staticmethod
    def backward(ctx, *gs):
        mod = ctx.mod
        n = len(mod.out_features)
        ab = ctx.saved_tensors
        A, B = ab[:n], ab[n:]
        r = A[0].shape[0]
        s = mod.scaling
        dA, dB, dhs, grads = [], [], [], []
        zero = ab[0].new_zeros(1)
        for i in range(n):
            g = gs[i].reshape(-1, mod.out_features[i]).to(BF16)
            if not g.is_contiguous():
                g = g.contiguous()
            grads.append(g)
            dh = torch.addmm(zero, g, B[i], beta=0.0, alpha=s)    # [M, r]
            dhs.append(dh)
            dB.append(torch.addmm(zero, g.t(), ctx.h_all[:, i * r:(i + 1) * r], beta=0.0, alpha=s))
        dh_all = dhs[0] if n == 1 else torch.cat(dhs, dim=1)         # [M, n*r]
        # dA_i = dh_i^T @ x_hat: the projections of a group read the same saved activation, so their dh go through
        # the weight-gradient kernel side by side (32 output rows per call, the widest its LoRA-shaped form takes)
        # and x_hat is decoded once per call instead of once per projection
        per_call = max(1, 32 // r) * r
        for c0 in range(0, n * r, per_call):
            block = K.gradw_gemm(dh_all[:, c0:c0 + per_call], ctx.saved_x, out_dtype=A[0].dtype)
            dA.extend(block[j:j + r] for j in range(0, block.shape[0], r))
        # dX: all rank-r terms as one thin GEMM, then each base GEMM accumulates onto it in its epilogue
        dx = dh_all @ (A[0] if n == 1 else torch.cat(list(A), dim=0))
        w_all = K.nf4_dequantize(mod.base_all)
        row = 0
        for i, out in enumerate(mod.out_features):
            dx.addmm_(grads[i], w_all[row:row + out])
            row += out
        del w_all, grads, dhs
        ctx.h_all = None
        ctx.saved_x = None
        return (dx.reshape(gs[0].shape[:-1] + (mod.in_features,)), None, None) + tuple(dA) + tuple(dB)


# ---- attention -----------------------------------------------------------------------------------------------
def rope_tables(S, head_dim, theta, device):
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32, device=device) / head_dim))
    freqs = torch.outer(torch.arange(S, dtype=torch.float32, device=device), inv)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(BF16), emb.sin().to(BF16)


class CompressedAttention(torch.nn.Module):
    """RoPE, softmax(q @ k^T / sqrt(hd) + causal mask) @ v on the [B, S, H] projections, with q, k (after RoPE) and v
    saved as codes in the [B*S, nh*hd] layout and the probabilities saved once as the entries above a calibrated
    threshold.  Composition of apply_rotary_pos_emb and the reference's gemm1, softmax and gemm2 modules
    (models/modeling_llama.py:423-462, operators/efficient_gemm.py, operators/efficient_softmax.py)."""

    def __init__(self, cfg: LayerConfig):
        super().__init__()
        if cfg.attention not in ("eager", "flash"):
            raise ValueError("attention must be 'eager' or 'flash', got %r" % (cfg.attention,))
        self.cfg = cfg
        mk = lambda: CompressionSite(cfg.outlier_ratio, 1.0, cfg.act_bits, "per-token", 0, "hyc", cfg.act_group,
                                     cfg.scale_rule)
        self.site_q, self.site_k, self.site_v, self.site_o = mk(), mk(), mk(), mk()
        self.iteration = 0
        self.static_value = None          # probability threshold, as in EfficientMemorySoftmax
        self.record = None

    def forward(self, q, k, v, cos, sin):
        func = _FlashAttentionFunc if self.cfg.attention == "flash" else _AttentionFunc
        return func.apply(q, k, v, cos, sin, self)


def _matrices_per_group(total, s, budget_bytes):
    """[S, S] bf16 score matrices per group: within the budget, and the groups of equal size"""
    most = max(1, min(total, budget_bytes // (2 * s * s)))
    groups = -(-total // most)
    return -(-total // groups)


class _AttentionFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cos, sin, mod):
        cfg = mod.cfg
        b, s, H = q.shape
        nh, hd = cfg.heads, cfg.head_dim
        scale = 1.0 / math.sqrt(hd)
        # one pass per tensor: rotate, and write both the head-major copy the batched GEMMs need and the rows that
        # are compressed
        qh, q_rows = K.rope_to_heads(q, nh, cos, sin, want_rows=True)
        kh, k_rows = K.rope_to_heads(k, nh, cos, sin, want_rows=True)
        v_rows = v                                                # possibly a column slice of the fused projection
        vh = K.rope_to_heads(v_rows, nh)
        # The [S, S] score matrices are processed in groups that bound the transient tensors (they stay in
        # the last-level cache and the peak memory no longer grows with B * heads): per group one library GEMM for
        # scores = (q @ k^T) / sqrt(hd), the softmax kernel with the causal mask built in (the masked half is never
        # read; the probabilities overwrite the scores), one GEMM for p @ v.
        q3, k3, v3 = qh.view(b * nh, s, hd), kh.view(b * nh, s, hd), vh.view(b * nh, s, hd)
        group = _matrices_per_group(b * nh, s, cfg.attn_group_bytes)
        it = mod.iteration
        calibrating = cfg.compress and it < 2
        if calibrating:
            group = b * nh                 # the threshold is a quantile over batch element 0: all of it is needed
        zero = q.new_zeros(1)
        out3 = torch.empty_like(q3)
        kept, p_all = [], None
        for c0 in range(0, b * nh, group):
            c1 = min(c0 + group, b * nh)
            scores = torch.baddbmm(zero, q3[c0:c1], k3[c0:c1].transpose(1, 2), beta=0.0, alpha=scale)
            if not cfg.compress:
                p, _ = K.softmax_fwd(scores, causal_period=s, inplace=True)
                kept.append(p)                                     # kept whole, in bf16
            elif not calibrating:
                p, sp = K.softmax_fwd(scores, K.threshold_value(mod.static_value), causal_period=s, inplace=True,
                                      budget=K.kept_budget(mod.static_value))
                kept.append(sp)
            else:
                p, _ = K.softmax_fwd(scores, causal_period=s, inplace=True)
                thr = get_statistics_softmax(p.view(b, nh, s, s), it, cfg.softmax_ratio)
                mod.static_value = running_mean(mod.static_value, thr, it)
                kept.append(K.softmax_sparsify(p, K.threshold_value(thr)))
            del scores
            torch.bmm(p, v3[c0:c1], out=out3[c0:c1])
            if mod.record is not None:
                p_all = p if p_all is None else torch.cat([p_all, p])
            del p
        out = K.rope_from_heads(out3.view(b, nh, s, hd))            # [B, S, H]
        del qh, kh, vh, q3, k3, v3, out3
        rows = [t.reshape(b * s, H) for t in (q_rows, k_rows, v_rows)]      # views (v keeps its pitch)
        if cfg.compress:
            saved = []
            for site, r in zip((mod.site_q, mod.site_k, mod.site_v), rows):
                plan = site.channel_plan(r, it)
                saved.append(K.compress_channel(r, plan, cfg.act_bits, cfg.act_group))
        else:
            saved = [r.contiguous() for r in rows]
        mod.iteration += 1
        if mod.record is not None:
            mod.record.update(q=rows[0].detach().clone(), k=rows[1].detach().clone(), v=rows[2].detach().clone(),
                              p=p_all.view(b, nh, s, s), saved=saved, sparse=list(kept))
        ctx.saved, ctx.kept, ctx.group, ctx.geom, ctx.compress = saved, kept, group, (b, nh, s, hd), cfg.compress
        ctx.save_for_backward(cos, sin)
        return out

    @staticmethod
    def backward(ctx, g):
        b, nh, s, hd = ctx.geom
        cos, sin = ctx.saved_tensors
        restore = (lambda c: K.decompress_channel(c)) if ctx.compress else (lambda c: c)
        to_heads = lambda rows: K.rope_to_heads(rows.view(b, s, nh * hd), nh).view(b * nh, s, hd)
        gh = K.rope_to_heads(g.to(BF16).contiguous(), nh).view(b * nh, s, hd)
        v = to_heads(restore(ctx.saved[2]))
        kk = to_heads(restore(ctx.saved[1]))
        qq = to_heads(restore(ctx.saved[0]))
        dq, dk, dv = torch.empty_like(qq), torch.empty_like(qq), torch.empty_like(qq)
        scale = 1.0 / math.sqrt(hd)
        zero = gh.new_zeros(1)                                     # ignored (beta = 0), only has to broadcast
        for i, c0 in enumerate(range(0, b * nh, ctx.group)):
            c1 = min(c0 + ctx.group, b * nh)
            item = ctx.kept[i]
            p = K.softmax_dense(item) if ctx.compress else item
            torch.bmm(p.transpose(1, 2), gh[c0:c1], out=dv[c0:c1])
            dp = torch.bmm(gh[c0:c1], v[c0:c1].transpose(1, 2))
            if ctx.compress:
                del p
                ds = K.softmax_bwd(dp, item, inplace=True)
            else:
                ds = torch._softmax_backward_data(dp, p, -1, BF16)
                del p
            del dp
            torch.baddbmm(zero, ds, kk[c0:c1], beta=0.0, alpha=scale, out=dq[c0:c1])
            torch.baddbmm(zero, ds.transpose(1, 2), qq[c0:c1], beta=0.0, alpha=scale, out=dk[c0:c1])
            del ds
            ctx.kept[i] = None
        del v, kk, qq, gh
        ctx.saved = ctx.kept = None
        dq = K.rope_from_heads(dq.view(b, nh, s, hd), cos, sin)
        dk = K.rope_from_heads(dk.view(b, nh, s, hd), cos, sin)
        dv = K.rope_from_heads(dv.view(b, nh, s, hd))
        return dq, dk, dv, None, None, None


class _FlashAttentionFunc(torch.autograd.Function):
    """The design of the reference's flash-attention operator (operators/efficient_flashattention.py:10-135): the
    fused attention kernel of the library runs the forward, what is kept is q, k (after RoPE), v and the attention
    output as codes plus the fp32 log-sum-exp of every row, and the library's backward kernel runs on the restored
    tensors.  No [S, S] matrix exists at any time.  The backward kernel rebuilds the probabilities from the restored
    q and k with the exact log-sum-exp, and takes its row term sum(dO * O) from the restored output."""

    @staticmethod
    def forward(ctx, q, k, v, cos, sin, mod):
        cfg = mod.cfg
        b, s, H = q.shape
        nh, hd = cfg.heads, cfg.head_dim
        scale = 1.0 / math.sqrt(hd)
        qh, q_rows = K.rope_to_heads(q, nh, cos, sin, want_rows=True)
        kh, k_rows = K.rope_to_heads(k, nh, cos, sin, want_rows=True)
        vh = K.rope_to_heads(v, nh)
        out_h, lse, _, _, _, _, seed, offset, _ = torch.ops.aten._scaled_dot_product_flash_attention(
            qh, kh, vh, 0.0, True, False, scale=scale)
        del qh, kh, vh
        out = K.rope_from_heads(out_h)                              # [B, S, H]
        del out_h
        rows = [t.reshape(b * s, H) for t in (q_rows, k_rows, v, out)]
        it = mod.iteration
        if cfg.compress:
            saved = []
            for site, r in zip((mod.site_q, mod.site_k, mod.site_v, mod.site_o), rows):
                saved.append(K.compress_channel(r, site.channel_plan(r, it), cfg.act_bits, cfg.act_group))
        else:
            saved = [r.contiguous() for r in rows]
        mod.iteration += 1
        if mod.record is not None:
            mod.record.update(q=rows[0].detach().clone(), k=rows[1].detach().clone(), v=rows[2].detach().clone(),
                              o=rows[3].detach().clone(), saved=saved, lse=lse)
        ctx.saved, ctx.geom, ctx.compress, ctx.rng = saved, (b, nh, s, hd), cfg.compress, (seed, offset)
        ctx.save_for_backward(cos, sin, lse)
        return out

    @staticmethod
    def backward(ctx, g):
        b, nh, s, hd = ctx.geom
        cos, sin, lse = ctx.saved_tensors
        restore = (lambda c: K.decompress_channel(c)) if ctx.compress else (lambda c: c)
        to_heads = lambda rows: K.rope_to_heads(rows.view(b, s, nh * hd), nh)
        gh = K.rope_to_heads(g.to(BF16).contiguous(), nh)
        qq, kk, vv, oo = (to_heads(restore(c)) for c in ctx.saved)
        ctx.saved = None
        dq, dk, dv = torch.ops.aten._scaled_dot_product_flash_attention_backward(
            gh, qq, kk, vv, oo, lse, None, None, s, s, 0.0, True, ctx.rng[0], ctx.rng[1], scale=1.0 / math.sqrt(hd))
        del gh, qq, kk, vv, oo
        dq = K.rope_from_heads(dq.contiguous(), cos, sin)
        dk = K.rope_from_heads(dk.contiguous(), cos, sin)
        dv = K.rope_from_heads(dv.contiguous())
        return dq, dk, dv, None, None, None


# ---- the layer --------------------------------------------------------------------------------------------------
class _PlainRMSNorm(torch.nn.Module):
    def __init__(self, hidden, eps, device):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.ones(hidden, dtype=BF16, device=device))
        self.eps = eps

    def forward(self, x):
        xf = x.float()
        return (self.weight.float() * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps))).to(x.dtype)


class DecoderLayer(torch.nn.Module):
    def __init__(self, cfg: LayerConfig = None, device="cuda"):
        super().__init__()
        self.cfg = cfg = cfg or LayerConfig()
        H, I = cfg.hidden, cfg.intermediate
        if cfg.heads * cfg.head_dim != H:
            raise ValueError("heads * head_dim must equal hidden")
        if cfg.compress:
            norm = lambda: EfficientMemoryRMSNorm(H, eps=cfg.rms_eps, elementwise_affine=True, bias=False,
                                                  outlier_ratio=cfg.outlier_ratio, sub_outlier_ratio=1.0,
                                                  sub_outlier_bit=cfg.act_bits, sub_outlier_quantize_method="per-token",
                                                  rank=0, mode="hyc", group_size=cfg.act_group,
                                                  scale_rule=cfg.scale_rule).to(device).to(BF16)
        else:
            norm = lambda: _PlainRMSNorm(H, cfg.rms_eps, device)
        self.input_layernorm = norm()
        self.post_attention_layernorm = norm()
        self.qkv_proj = LoRAProjections(H, [H, H, H], cfg, device)
        self.o_proj = LoRAProjections(H, [H], cfg, device)
        self.gate_up_proj = LoRAProjections(H, [I, I], cfg, device)
        self.down_proj = LoRAProjections(I, [H], cfg, device)
        self.attention = CompressedAttention(cfg)
        self.act = EfficientMemoryGatedAct("silu", cfg.outlier_ratio, 1.0, cfg.act_bits, "per-token", 0,
                                           group_size=cfg.act_group, scale_rule=cfg.scale_rule) if cfg.compress else None
        self._rope = None

    def forward(self, x):
        cfg = self.cfg
        b, s, H = x.shape
        if self._rope is None or self._rope[0].shape[0] != s:
            self._rope = rope_tables(s, cfg.head_dim, cfg.rope_theta, x.device)
        cos, sin = self._rope
        # no names for the wide intermediates: each is released as soon as its consumer has run
        x = x + self.o_proj(self.attention(*self.qkv_proj(self.input_layernorm(x)), cos, sin))
        return x + self.down_proj(self._gated(*self.gate_up_proj(self.post_attention_layernorm(x))))

    def _gated(self, gate, up):
        if self.act is not None:
            return self.act(gate, up)
        return torch.nn.functional.silu(gate) * up

    def saved_activation_bytes(self, batch, seq):
        """analytic size of what one forward keeps for the backward (the probabilities' share is data dependent:
        `softmax_ratio` of B*nh*S*S entries of 6 bytes plus row pointers; the fused attention keeps its output and
        one fp32 log-sum-exp per row instead)"""
        cfg = self.cfg
        M, H, I = batch * seq, cfg.hidden, cfg.intermediate

        def site(width, bits, group):
            k = K.num_outlier_channels(width, cfg.outlier_ratio)
            return M * (width * bits // 8 + 2 * k + 2 * (width // group))

        total = 2 * (site(H, cfg.act_bits, cfg.act_group) + 4 * M)                    # two norms: x + rstd
        total += 2 * site(H, cfg.linear_bits, cfg.linear_group)                       # qkv input (once), o input
        total += site(H, cfg.linear_bits, cfg.linear_group) + site(I, cfg.linear_bits, cfg.linear_group)  # gate/up, down
        total += 3 * site(H, cfg.act_bits, cfg.act_group)                             # q, k, v
        total += 3 * site(I, cfg.act_bits, cfg.act_group)                             # gate, act(gate), up
        total += 7 * M * cfg.lora_r * 2                                               # h = x @ A^T, exact
        rows = batch * cfg.heads * seq
        if cfg.attention == "flash":
            total += site(H, cfg.act_bits, cfg.act_group) + 4 * rows                  # attention output, log-sum-exp
        else:
            total += int(cfg.softmax_ratio * rows * seq) * 6 + 4 * (rows + 1)
        return total
