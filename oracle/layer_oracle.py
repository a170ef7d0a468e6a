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


def decoder_layer(x, params, restored, nh, eps, scaling, cos, sin, quirk=True, probs=None, capture=None):
    """x fp32 [B,S,H] (requires_grad); params: dict of fp32 tensors W_q.. (dequantised), A_q.., B_q.., w_in, w_post;
    restored: dict site -> x_hat for sites norm_in, qkv_in, q, k, v, p, o_in, norm_post, gate_up_in, gate, act, up,
    down_in (q, k, v in the [B,S,H] layout, p [B,nh,S,S]); a site that is missing keeps its exact activation.
    `probs`, when given, replaces the recomputed softmax value (a caller that holds the device's probabilities passes
    them so that p_hat and p agree).  `capture`, when a dict, receives the exact activation of every site."""
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
    scores = _value_of(q @ k.transpose(-2, -1), _st(q, q_hat) @ _st(k, k_hat).transpose(-2, -1))
    scores = scores / math.sqrt(q.shape[-1])
    mask = torch.ones(s, s, dtype=torch.bool).triu(1)
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
