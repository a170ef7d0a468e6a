"""CPU oracle of one LoRA decoder layer whose backward sees compressed activations.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE (see hyc_oracle.py).

The layer is the reference's swapped LLaMA layer (models/modeling_llama.py:263-295 MLP, :382-484 attention,
:786-845 layer; peft LoRA around a 4-bit base, bitsandbytes_fix/_function.py:509-540) written with plain torch
autograd in fp32.  Every operator the reference swaps keeps its exact forward value and takes its backward from
the restored activation x_hat, exactly as the operators' backward functions do:

    linear   dA = dh^T @ x_hat                                   operators/efficient_linear.py:56-67
    rmsnorm  hyc_oracle.rmsnorm_bwd at x_hat (with the c2 term)  operators/efficient_rmsnorm.py:63-143
    silu     silu'(gate_hat) * g                                 operators/efficient_silu.py:44-53
    product  g * up_hat, act_hat * g                             operators/efficient_hadamard.py:55-83
    q @ kT   g @ kT_hat^T, q_hat^T @ g                           operators/efficient_gemm.py:64-78
    softmax  (g - sum(g * p_hat)) * p_hat                        operators/efficient_softmax.py:37-45
    p @ v    g @ v_hat^T, p_hat^T @ g                            operators/efficient_gemm.py:232-240
    fused attention (attention="flash"): the flash-attention backward evaluated at q_hat, k_hat, v_hat, o_hat with
             the exact log-sum-exp of the forward                operators/efficient_flashattention.py:97-134

`restored` maps a site name to x_hat.  Pinning: with x_hat = x every formula above is the true derivative, so the
whole layer is checked against torch.autograd of the same layer without substitution (tests/test_oracle_pins.py);
rmsnorm_bwd and the elementwise formulas have their own pins in hyc_oracle.py.  The reference's models/ cannot run
here (peft, bitsandbytes and a GPU are needed): PARITY UNPINNED by reference outputs at the layer level.
"""
import math

import torch

from . import hyc_oracle as O


def _st(x, x_hat):
    """value x_hat, gradient passed straight to x"""
    return x + (x_hat.to(x.dtype) - x).detach()


def _value_of(exact, through):
    """value `exact`, gradient of `through`"""
    return through + (exact - through).detach()


class _RMSNormAt(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, eps, x_hat, quirk):
        y, rstd = O.rmsnorm_fwd(x.to(O.BF16), w, eps)
        ctx.save_for_backward(x_hat, w, rstd)
        ctx.quirk = quirk
        return y.float()

    @staticmethod
    def backward(ctx, dy):
        x_hat, w, rstd = ctx.saved_tensors
        dx, dw = O.rmsnorm_bwd(dy.to(O.BF16), x_hat.to(O.BF16), w, rstd, c2_quirk=ctx.quirk)
        return dx.float(), dw.float(), None, None, None


class _SoftmaxAt(torch.autograd.Function):
    @staticmethod
    def forward(ctx, s, p_hat):
        ctx.save_for_backward(p_hat)
        return torch.softmax(s, dim=-1)

    @staticmethod
    def backward(ctx, g):
        (p_hat,) = ctx.saved_tensors
        return O.softmax_bwd(p_hat.float(), g), None


class _FlashAttentionAt(torch.autograd.Function):
    """Causal attention whose backward is the flash-attention backward pass run on restored tensors, as the
    reference does when it hands decompressed q, k, v, out and the saved softmax_lse to _flash_attn_varlen_backward
    (operators/efficient_flashattention.py:97-134).  That pass never sees the forward's probabilities: it rebuilds
    P_hat = exp(q_hat k_hat^T * scale - lse) with the exact log-sum-exp (so P_hat's rows need not sum to one), takes
    the row term D = sum(dO * o_hat) from the restored output, and forms
        dV = P_hat^T dO,  dP = dO v_hat^T,  dS = P_hat * (dP - D),  dQ = scale * dS k_hat,  dK = scale * dS^T q_hat.
    With every restored tensor equal to the exact one this is the true derivative (D = sum_j P_ij dP_ij)."""

    @staticmethod
    def forward(ctx, q, k, v, q_hat, k_hat, v_hat, o_hat, scale, causal=True):
        s = q.shape[-2]
        mask = (torch.ones(s, s, dtype=torch.bool, device=q.device).triu(1) if causal else
                torch.zeros(s, s, dtype=torch.bool, device=q.device))
        scores = (q @ k.transpose(-2, -1)) * scale
        scores = scores.masked_fill(mask, float("-inf"))
        lse = torch.logsumexp(scores, dim=-1, keepdim=True)
        ctx.save_for_backward(q_hat, k_hat, v_hat, o_hat, lse, mask)
        ctx.scale = scale
        return torch.exp(scores - lse) @ v

    @staticmethod
    def backward(ctx, g):
        q_hat, k_hat, v_hat, o_hat, lse, mask = ctx.saved_tensors
        scores = ((q_hat @ k_hat.transpose(-2, -1)) * ctx.scale).masked_fill(mask, float("-inf"))
        p_hat = torch.exp(scores - lse)
        dv = p_hat.transpose(-2, -1) @ g
        dp = g @ v_hat.transpose(-2, -1)
        d = (g * o_hat).sum(-1, keepdim=True)
        ds = p_hat * (dp - d)
        dq = ctx.scale * (ds @ k_hat)
        dk = ctx.scale * (ds.transpose(-2, -1) @ q_hat)
        return dq, dk, dv, None, None, None, None, None, None


def lora_projection(x, x_hat, W, A, B, scaling):
    """y = x W^T + s (x A^T) B^T; dA from x_hat, dB from the exact h"""
    h = _value_of(x @ A.t(), _st(x, x_hat) @ A.t())
    return x @ W.t() + scaling * (h @ B.t())


def rotate_half(x):
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def rope(x, cos, sin):
    return x * cos + rotate_half(x) * sin


def heads(x, nh):
    b, s, H = x.shape
    return x.view(b, s, nh, H // nh).transpose(1, 2)


def rows(x):
    """[B,nh,S,hd] -> [B,S,nh*hd]"""
    b, nh, s, hd = x.shape
    return x.transpose(1, 2).reshape(b, s, nh * hd)


def decoder_layer(x, params, restored, nh, eps, scaling, cos, sin, quirk=True, probs=None, capture=None,
                  attention="eager"):
    """x fp32 [B,S,H] (requires_grad); params: dict of fp32 tensors W_q.. (dequantised), A_q.., B_q.., w_in, w_post;
    restored: dict site -> x_hat for sites norm_in, qkv_in, q, k, v, p, o_in, norm_post, gate_up_in, gate, act, up,
    down_in (q, k, v in the [B,S,H] layout, p [B,nh,S,S]); a site that is missing keeps its exact activation.
    `probs`, when given, replaces the recomputed softmax value (a caller that holds the device's probabilities passes
    them so that p_hat and p agree).  `capture`, when a dict, receives the exact activation of every site.
    attention="flash": no site p; instead site o, the attention output in the [B,S,H] layout."""
    P = params

    def hat(name, exact):
        if capture is not None:
            capture[name] = exact.detach().clone()
        got = restored.get(name)
        return exact.detach() if got is None else got.float()

    b, s, H = x.shape
    h = _RMSNormAt.apply(x, P["w_in"], eps, hat("norm_in", x), quirk)
    h_hat = hat("qkv_in", h)
    q, k, v = (lora_projection(h, h_hat, P["W_" + n], P["A_" + n], P["B_" + n], scaling) for n in "qkv")
    q, k, v = rope(heads(q, nh), cos, sin), rope(heads(k, nh), cos, sin), heads(v, nh)
    q_hat, k_hat, v_hat = (heads(hat(n, rows(t)), nh) for n, t in (("q", q), ("k", k), ("v", v)))
    if attention == "flash":
        with torch.no_grad():
            mask = torch.ones(s, s, dtype=torch.bool, device=q.device).triu(1)
            sc = (q @ k.transpose(-2, -1) / math.sqrt(q.shape[-1])).masked_fill(mask, float("-inf"))
            o_exact = rows(torch.softmax(sc, dim=-1) @ v)
        o_hat = heads(hat("o", o_exact), nh)
        a = rows(_FlashAttentionAt.apply(q, k, v, q_hat, k_hat, v_hat, o_hat, 1.0 / math.sqrt(q.shape[-1])))
    else:
        scores = _value_of(q @ k.transpose(-2, -1), _st(q, q_hat) @ _st(k, k_hat).transpose(-2, -1))
        scores = scores / math.sqrt(q.shape[-1])
        mask = torch.ones(s, s, dtype=torch.bool, device=q.device).triu(1)
        scores = scores.masked_fill(mask, torch.finfo(torch.bfloat16).min)
        p_exact = torch.softmax(scores.detach(), dim=-1) if probs is None else probs.float()
        p_hat = hat("p", p_exact)
        p = _value_of(p_exact, _SoftmaxAt.apply(scores, p_hat))
        a = _value_of(p @ v, _st(p, p_hat) @ _st(v, v_hat))
        a = rows(a)
    x1 = x + lora_projection(a, hat("o_in", a), P["W_o"], P["A_o"], P["B_o"], scaling)
    h2 = _RMSNormAt.apply(x1, P["w_post"], eps, hat("norm_post", x1), quirk)
    h2_hat = hat("gate_up_in", h2)
    gate = lora_projection(h2, h2_hat, P["W_gate"], P["A_gate"], P["B_gate"], scaling)
    up = lora_projection(h2, h2_hat, P["W_up"], P["A_up"], P["B_up"], scaling)
    act_exact = torch.nn.functional.silu(gate)
    act = _value_of(act_exact, torch.nn.functional.silu(_st(gate, hat("gate", gate))))
    m = _value_of(act * up, _st(act, hat("act", act_exact)) * _st(up, hat("up", up)))
    return x1 + lora_projection(m, hat("down_in", m), P["W_down"], P["A_down"], P["B_down"], scaling)
