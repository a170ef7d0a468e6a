"""CPU oracle for the HyC-LoRA hybrid activation-compression hot path.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests, the smoke check and
the benchmark's cpu-baseline leg may import it; the product package never does.

Everything here is a restatement, on CPU PyTorch tensors, of the arithmetic the
reference performs (same op order, same dtypes, hence the same bf16 roundings).
Each function cites the reference lines it follows.  Two families:

* ``ref_*``  - the scheme the reference snapshot implements: element-threshold
  outliers kept as a COO sparse tensor, a static scale (per-tensor / per-channel
  / per-token), an optional rank-r base ``L @ R``.
* ``hyc_*``  - the channel-structured variant: the k channels with the largest
  per-channel abs-max are kept verbatim as a dense ``[M, k]`` side tensor, the
  rest is quantised with a scale per (token, group of G channels).  The reference
  holds no implementation of the channel selection rule; the functions below are
  composed from the reference's primitives (zero-out, divide, round, clamp,
  offset, half-split packing).  Quantise / pack / unpack / dequantise are shared
  with the ``ref_*`` family and pinned with it; the group scales (both rules, see
  hyc_group_scales) are pinned by an integer model, invariants and the special case
  that reduces to the reference's per-token scheme (below).  The selection rule has
  no counterpart in the reference to pin against.

Pinning status (see tests/test_oracle_*.py):
* pack / unpack                - brute force over all byte values, pure Python loops
* quantise                     - all 65536 bf16 patterns x scales vs exact rationals
* ref_compress / ref_decompress / get_statistics / softmax helpers / SiLU, GELU,
  Hadamard, softmax backward / calibration protocol
                               - golden vectors written by importing the reference
* rmsnorm_fwd / rmsnorm_bwd    - closed form + torch.autograd (reference kernels are
                                 Triton and cannot run without a GPU)
* layernorm_fwd / layernorm_bwd - torch's own layer norm + float64 torch.autograd (reference
                                 kernels are Triton): parity unpinned by reference outputs
* linear_bwd                   - torch.matmul in fp32
* gemm_bwd                     - torch.autograd of torch.matmul in float64
* rope_fwd / rope_bwd          - complex-number form of the rotation; float64 torch.autograd
* philox4x32_10 / dropout_*    - Random123 known-answer vectors for the generator; keep fraction; the mask
                                 mapping itself restates triton 3.6.0's tl.rand: parity unpinned by reference outputs
* hyc group scales (hyc_group_scales, rules "range" and "absmax")
                               - integer model of bf16(bf16(a) / levels) in exact rationals with round-half-even
                                 on tiny inputs; range rule: a group's min and max land 2^b - 1 codes apart (+-1);
                                 absmax rule: the extreme element takes the extreme code and every element is
                                 within half a step; group = H, k = 0 with the range rule = ref_compress with the
                                 golden-pinned per-token scale, byte for byte
* hyc_select_channels          - brute force on small inputs, ties, idempotence; no reference code exists for the
                                 channel rule, so there are no reference outputs to pin it to
* nf4_quantize / nf4_dequantize - parity unpinned (bitsandbytes is not in the reference tree); checked against
                                 the published level table: nearest level by exact distance, round trips
"""
import math

import torch

BF16 = torch.bfloat16


# --------------------------------------------------------------------------------------
# shape helpers                                  operators/compress_function.py:4-12
# --------------------------------------------------------------------------------------
def hidden_to_head_shape(x, num_heads):
    b, s, h = x.shape
    return x.reshape(b, s, num_heads, h // num_heads).transpose(1, 2)


def head_to_hidden_shape(x):
    b, nh, s, hd = x.shape
    return x.transpose(1, 2).reshape(b, s, nh * hd)


def pad_cut_L(src_L, tgt_L):
    """Zero-pad or cut the rows of src_L to the row count of tgt_L.
    operators/compress_function.py:350-360"""
    have, r = src_L.shape
    want = tgt_L.shape[0]
    if have < want:
        pad = torch.zeros(want - have, r, dtype=src_L.dtype, device=src_L.device)
        src_L = torch.cat((src_L, pad), dim=0)
    elif have > want:
        src_L = src_L[:want, :]
    return src_L.contiguous()


# --------------------------------------------------------------------------------------
# bit packing                                     operators/compress_function.py:175-197, 218-255
# --------------------------------------------------------------------------------------
def pack_codes(codes_u8, bits):
    """codes_u8 [..., H] uint8 in [0, 2^bits) -> [..., H*bits/8] uint8.

    Segment layout: the last dim is cut into n = 8/bits equal segments; byte j holds
    segment i's element j in bit field [i*bits, (i+1)*bits).  (bits == 8 is not packed
    by the reference - it stores int8 - and is not handled here.)"""
    assert bits in (1, 2, 4)
    n = 8 // bits
    H = codes_u8.shape[-1]
    seg = H // n
    out = None
    # the reference adds the highest segment first; uint8 addition is commutative and
    # the fields are disjoint, so the order is immaterial.
    for i in range(n):
        part = codes_u8[..., i * seg:(i + 1) * seg] * (2 ** (i * bits))
        out = part if out is None else out + part
    return out


def unpack_codes(packed_u8, bits):
    """Inverse of pack_codes using the reference's %, -, // chain (:222-252)."""
    assert bits in (1, 2, 4)
    n = 8 // bits
    base = 2 ** bits
    rest = packed_u8
    parts = []
    for i in range(n):
        if i < n - 1:
            low = rest % base
            rest = (rest - low) // base
            parts.append(low)
        else:
            parts.append(rest)
    return torch.cat(parts, dim=-1)


# --------------------------------------------------------------------------------------
# quantise / dequantise primitives              operators/compress_function.py:170, 221-255
# --------------------------------------------------------------------------------------
def quantize_q(x, scale, bits, define_nan=False):
    """q = clamp(round(x / scale), -2^(b-1), 2^(b-1)-1); x, scale bf16 (broadcastable).

    The division result is a bf16 tensor (fp32 divide rounded to nearest even), round is
    half-to-even, then the clamp.  0/0 gives NaN, whose cast to an integer type the reference
    leaves to the platform; with define_nan those positions get q = 0 (what the HIP kernels do)."""
    off = 2 ** (bits - 1)
    q = torch.clamp(torch.round(x / scale), min=-off, max=off - 1)
    if define_nan:
        q = torch.where(torch.isnan(q), torch.zeros_like(q), q)
    return q


def encode_q(q, bits):
    """q (bf16 integers) -> stored tensor: int8 for 8 bits, packed uint8 otherwise."""
    if bits == 8:
        return q.to(torch.int8)
    off = 2 ** (bits - 1)
    return pack_codes((q + off).to(torch.uint8), bits)


def decode_stored(stored, bits, scale, dtype=BF16):
    """stored -> dequantised bf16 ((code - off) * scale, each op rounding to bf16)."""
    if bits == 8:
        return stored.to(dtype) * scale
    off = 2 ** (bits - 1)
    return (unpack_codes(stored, bits).to(dtype) - off) * scale


# --------------------------------------------------------------------------------------
# calibration                                    operators/compress_function.py:292-347
# --------------------------------------------------------------------------------------
@torch.no_grad()
def get_statistics(x, iteration, outlier_ratio, sub_outlier_ratio, sub_outlier_bit=8,
                   sub_outlier_quantize_method='per-tensor', svd_rank=16):
    """Threshold, rank-r base and static scale from batch element 0.
    Returns (thr f32 0-d, L bf16 [S,r], R bf16 [r,H], scale bf16)."""
    if x.dim() == 4:
        b, nh, s, hd = x.shape
        x = x.permute(0, 2, 1, 3).reshape(b, s, nh * hd)
    if svd_rank > 0:
        U, S, V = torch.svd_lowrank(x[0].to(torch.float32), q=svd_rank, niter=16)
        L = U.contiguous()
        R = (torch.diag(S) @ V.T).contiguous()
        x = x - L @ R                       # promotes x to fp32 from here on
    else:
        L = torch.zeros((x.shape[-2], 16), dtype=x.dtype, device=x.device)
        R = torch.zeros((16, x.shape[-1]), dtype=x.dtype, device=x.device)

    first = x[0]
    kth = int(first.numel() * (1 - outlier_ratio))
    thr = torch.kthvalue(first.flatten().to(torch.float32), kth).values     # signed quantile
    big = (first * (first.abs() > thr)).to(BF16)
    x = x - big                             # batch 0's outliers, broadcast over the batch

    if sub_outlier_ratio > 0 and sub_outlier_bit != 16:
        z = x[0]
        levels = 2 ** sub_outlier_bit - 1
        if sub_outlier_quantize_method == 'per-tensor':
            scale = (z.max() - z.min()) / levels
        elif sub_outlier_quantize_method == 'per-channel':
            scale = (z.max(dim=-2, keepdim=True).values - z.min(dim=-2, keepdim=True).values) / levels
        elif sub_outlier_quantize_method == 'per-token':
            scale = (z.max(dim=-1, keepdim=True).values - z.min(dim=-1, keepdim=True).values) / levels
        else:
            raise ValueError("Unsupport Quantize Method")
    else:
        scale = torch.tensor(1., device=x.device)
    return thr, L.to(BF16), R.to(BF16), scale.to(BF16)


@torch.no_grad()
def get_statistics_softmax(y, iteration, outlier_ratio):
    """operators/compress_function.py:343-347"""
    first = y[0]
    return torch.kthvalue(first.float().flatten(), int(first.numel() * (1 - outlier_ratio))).values


def running_mean_update(static, fresh, iteration):
    """One step of the modules' calibration average, e.g. operators/efficient_silu.py:86-111.
    static / fresh are [thr, L, scale, R] lists (note the order)."""
    if iteration >= 2:
        return static
    out = list(static)
    for slot in range(4):
        new = fresh[slot]
        if static[slot] is None:
            out[slot] = new
        else:
            if slot == 1:
                new = pad_cut_L(new, static[slot])
            out[slot] = (iteration * static[slot] + new) / (iteration + 1)
    return out


# --------------------------------------------------------------------------------------
# ref-mode compress / decompress                 operators/compress_function.py:136-261
# --------------------------------------------------------------------------------------
@torch.no_grad()
def ref_compress(x, thr, scale, bits=8, sub_outlier_ratio=1., L=None, R=None, define_nan=False):
    """-> (coo sparse bf16 of the outliers, stored codes, scale).  x is [B,S,H] or [B,nh,S,hd].
    define_nan=True replaces the platform-defined integer cast of 0/0 by q = 0 (see quantize_q)."""
    if x.dim() == 4:
        x = head_to_hidden_shape(x)
    S = x.shape[-2]
    base = pad_cut_L(L, torch.zeros((S, L.shape[-1]))) @ R          # bf16 matmul -> bf16
    x = x - base
    hot = x.abs() > thr                                             # thr rounds to x's dtype
    big = x * hot
    x = x - big                                                     # exact zeros at hot positions
    if torch.sum(scale) != 1.:
        big_c = big.to(BF16).to_sparse()
    else:
        big_c = big
    assert sub_outlier_ratio != 0., "the no-quantisation branch is not part of the path"
    assert bits in (1, 2, 4, 8), "bits must be 1, 2, 4 or 8 on this path"
    q = quantize_q(x, scale, bits, define_nan)
    return big_c, encode_q(q, bits), scale


@torch.no_grad()
def ref_decompress(big_c, stored, bits, scale, is_head=False, num_heads=1, L=None, R=None):
    big = big_c.to_dense() if big_c.is_sparse else big_c
    S = big.shape[-2]
    x = (pad_cut_L(L, torch.zeros((S, L.shape[-1]))) @ R).to(BF16)
    x = x + big
    if torch.sum(scale) != 1.:
        x = x + decode_stored(stored, bits, scale, big.dtype)
    if is_head:
        x = hidden_to_head_shape(x, num_heads)
    return x


# --------------------------------------------------------------------------------------
# softmax sparsification                          operators/compress_function.py:264-281
# --------------------------------------------------------------------------------------
def prune_softmax(y, thr):
    return y * (y > thr)


@torch.no_grad()
def true_compress_softmax(y, thr):
    return prune_softmax(y, thr).to_sparse()


@torch.no_grad()
def true_decompress_softmax(y_sparse):
    return y_sparse.to_dense()


# --------------------------------------------------------------------------------------
# low-rank helpers                                operators/fused_compression.py:5-67, 102-171
# --------------------------------------------------------------------------------------
def low_rank_extraction(l, r, x):
    """x[b] - l@r accumulated in fp32 from the bf16 operands, one rounding to bf16."""
    return (x.float() - (l.float() @ r.float())[None]).to(BF16)


def low_rank_addition(l, r, x):
    return (x.float() + (l.float() @ r.float())[None]).to(BF16)


# --------------------------------------------------------------------------------------
# hyc mode: channel outliers + per-(token, group) scales
# --------------------------------------------------------------------------------------
def hyc_num_outlier_channels(H, ratio):
    return int(math.floor(ratio * H + 0.5))


def hyc_channel_scores(x):
    """max over all tokens of |x[..., c]| - exact in bf16; returned as fp32 [H]."""
    return x.reshape(-1, x.shape[-1]).abs().amax(dim=0).float()


def hyc_select_channels(scores, k):
    """k largest scores, ties to the lower channel index, returned ascending (int32)."""
    order = torch.sort(scores, descending=True, stable=True).indices[:k]
    return torch.sort(order).values.to(torch.int32)


def hyc_group_scales(rest, bits, group, rule="absmax"):
    """bf16 [M, H/G] scales of the channel scheme from `rest` = x with the outlier channels zeroed.  No reference code
    exists for either rule; both are evaluated with the reference's arithmetic (bf16 tensor ops, each rounding to
    nearest even) and pinned in tests/test_oracle_pins.py by an integer-arithmetic model and by invariants.

    "range"   (max - min) / (2^b - 1): the reference's scale formula (compress_function.py:328-334) per token and
              group.  The codes have no zero point, so a group that is not centred on 0 clips at the code bounds.
    "absmax"  (2 max|x|) / (2^b - 1): the same formula over the interval made symmetric about zero,
              [-max|x|, max|x|]; every element lands within half a step of a code (1-bit codes, {-1, 0}: max|x|)."""
    M, H = rest.shape
    g = rest.reshape(M, H // group, group)
    if rule == "range":
        return (g.amax(dim=-1) - g.amin(dim=-1)) / (2 ** bits - 1)
    if rule == "absmax":
        am = g.abs().amax(dim=-1)
        return am if bits == 1 else (am + am) / (2 ** bits - 1)
    raise ValueError("rule must be 'range' or 'absmax'")


@torch.no_grad()
def hyc_compress(x, idx, bits, group, rule="absmax"):
    """x [M,H] bf16, idx [k] ascending -> (vals [M,k] bf16, stored, scales [M,H/G] bf16).

    Composition of the reference steps (:149-151 zero-out, :170 quantise, :175-197 pack) with
    the channel mask in place of the threshold mask and a scale per token and group of G channels
    (hyc_group_scales).  0/0 (an all-zero group) is given q = 0, i.e. code = offset."""
    M, H = x.shape
    idx = idx.long()
    hot = torch.zeros(H, dtype=torch.bool)
    hot[idx] = True
    big = x * hot
    vals = big[:, idx].contiguous()
    rest = x - big
    scales = hyc_group_scales(rest, bits, group, rule)
    q = quantize_q(rest.reshape(M, H // group, group), scales[..., None], bits, define_nan=True).reshape(M, H)
    return vals, encode_q(q, bits), scales


@torch.no_grad()
def hyc_decompress(vals, stored, idx, scales, bits, group):
    """-> x_hat [M,H] bf16 = (0 + scatter(vals)) + dequant (the order of :205-256)."""
    M = stored.shape[0]
    H = stored.shape[1] * (8 // bits)
    big = torch.zeros(M, H, dtype=BF16)
    big[:, idx.long()] = vals
    x = torch.zeros(M, H, dtype=BF16) + big
    sc = scales[..., None].expand(M, H // group, group).reshape(M, H)
    return x + decode_stored(stored, bits, sc)


# --------------------------------------------------------------------------------------
# RMSNorm                                         operators/efficient_rmsnorm.py:15-143
# --------------------------------------------------------------------------------------
def rmsnorm_fwd(x, w, eps):
    """fp32 math, one rounding: y = bf16((x * rstd) * w); rstd = 1/sqrt(mean(x^2) + eps).
    Returns (y in x's dtype, rstd fp32 [M])."""
    H = x.shape[-1]
    xf = x.reshape(-1, H).float()
    var = (xf * xf).sum(dim=-1) / H
    rstd = 1 / torch.sqrt(var + eps)
    y = ((xf * rstd[:, None]) * w.float()[None, :]).to(x.dtype)
    return y.reshape(x.shape), rstd


def rmsnorm_bwd(dy, x_hat, w, rstd, c2_quirk=True):
    """dx = (w*dy - (xn*c1 + c2)) * rstd with xn = x_hat*rstd, c1 = mean(xn*w*dy),
    c2 = mean(w*dy) (the reference keeps this LayerNorm term, :102-104; c2_quirk=False drops
    it, which is the true RMSNorm gradient).  dw = sum_rows dy*xn, accumulated in fp32 (the
    reference accumulates partials in a bf16 buffer in lock order, :107-119, so its dw is a
    noisier evaluation of the same sum).  Returns (dx bf16, dw in w's dtype)."""
    H = x_hat.shape[-1]
    xf = x_hat.reshape(-1, H).float()
    g = dy.reshape(-1, H).to(BF16).float()
    xn = xf * rstd[:, None]
    wdy = w.float()[None, :] * g
    c1 = (xn * wdy).sum(dim=-1, keepdim=True) / H
    c2 = wdy.sum(dim=-1, keepdim=True) / H if c2_quirk else 0.
    dx = ((wdy - (xn * c1 + c2)) * rstd[:, None]).to(BF16).reshape(dy.shape)
    dw = (g * xn).sum(dim=0).to(w.dtype)
    return dx, dw


# --------------------------------------------------------------------------------------
# LayerNorm                                      operators/efficient_layernorm.py:15-148
# --------------------------------------------------------------------------------------
def layernorm_fwd(x, w, b, eps):
    """two-pass statistics in fp32 (:27-41): mean, var = mean((x-mean)^2), rstd = 1/sqrt(var+eps);
    y = bf16(((x-mean)*rstd)*w + b) (:55-56).  Returns (y, mean fp32 [M], rstd fp32 [M])."""
    H = x.shape[-1]
    xf = x.reshape(-1, H).float()
    mean = xf.sum(dim=-1) / H
    xc = xf - mean[:, None]
    var = (xc * xc).sum(dim=-1) / H
    rstd = 1.0 / torch.sqrt(var + eps)
    y = (xc * rstd[:, None]) * w.float()[None, :]
    if b is not None:
        y = y + b.float()[None, :]
    return y.to(x.dtype).reshape(x.shape), mean, rstd


def layernorm_bwd(dy, x_hat, w, mean, rstd):
    """xhat = (x_hat-mean)*rstd; dx = (w*dy - (xhat*c1 + c2))*rstd, c1 = mean(xhat*w*dy), c2 = mean(w*dy) (:113-121);
    dw = sum_rows dy*xhat, db = sum_rows dy, accumulated in fp32 (the reference sums bf16 partials in lock order,
    :123-137).  Returns (dx bf16, dw, db in w's dtype)."""
    H = x_hat.shape[-1]
    xf = x_hat.reshape(-1, H).float()
    g = dy.reshape(-1, H).to(BF16).float()
    xn = (xf - mean[:, None]) * rstd[:, None]
    wdy = w.float()[None, :] * g
    c1 = (xn * wdy).sum(dim=-1, keepdim=True) / H
    c2 = wdy.sum(dim=-1, keepdim=True) / H
    dx = ((wdy - (xn * c1 + c2)) * rstd[:, None]).to(BF16).reshape(dy.shape)
    return dx, (g * xn).sum(dim=0).to(w.dtype), g.sum(dim=0).to(w.dtype)


# --------------------------------------------------------------------------------------
# activation / elementwise backward (bf16 op-by-op, as torch evaluates the expressions)
# --------------------------------------------------------------------------------------
def silu_bwd(x_hat, g):
    """operators/efficient_silu.py:50-51"""
    s = torch.sigmoid(x_hat)
    return s * (1 + x_hat - x_hat * s) * g


def gelu_bwd(x_hat, g):
    """tanh-form derivative, operators/efficient_gelu.py:49-62"""
    gamma = math.sqrt(2 / math.pi)
    kappa = 0.044715
    inner = gamma * (x_hat + kappa * x_hat ** 3)
    t = torch.tanh(inner)
    return 0.5 * ((1 + t) + x_hat * ((1 - t ** 2) * gamma * (1 + 3 * kappa * x_hat ** 2))) * g


def hadamard_bwd(x1_hat, x2_hat, g):
    """operators/efficient_hadamard.py:62-66"""
    return g * x2_hat, x1_hat * g


def softmax_bwd(y_hat, g):
    """operators/efficient_softmax.py:37-45"""
    return (g - (g * y_hat).sum(dim=-1, keepdims=True)) * y_hat


# --------------------------------------------------------------------------------------
# linear                                          operators/efficient_linear.py:56-83
# --------------------------------------------------------------------------------------
def linear_bwd(dy, x_hat, w, use_bias=False):
    """dX = dY @ W; dW = sum_b dY[b]^T @ x_hat[b] (the reference forms [B,out,in] in bf16 and
    autograd sum-reduces it over B); db = sum over every leading dim of dY.
    Returns (dX bf16, dW_literal bf16, dW_fp32 (single rounding-free reference), db or None)."""
    g = dy.to(w.dtype)
    dX = g @ w
    g2 = g.to(x_hat.dtype)
    per_batch = g2.transpose(-2, -1) @ x_hat
    dW_lit = per_batch.sum(0) if per_batch.dim() == 3 else per_batch
    out_f = dy.shape[-1]
    dW_f32 = g2.reshape(-1, out_f).float().t() @ x_hat.reshape(-1, x_hat.shape[-1]).float()
    db = g2.reshape(-1, out_f).float().sum(0).to(w.dtype) if use_bias else None
    return dX, dW_lit, dW_f32, db


# --------------------------------------------------------------------------------------
# attention products                              operators/efficient_gemm.py:64-78, 232-240
# --------------------------------------------------------------------------------------
def gemm_bwd(g, x1_hat, x2_hat):
    """y = x1 @ x2 with both operands restored from their compressed form:
    d_x1 = g @ x2_hat^T, d_x2 = x1_hat^T @ g (operators/efficient_gemm.py:72-73, 238-239), in fp32 so that the
    result carries no rounding of its own"""
    gf = g.float()
    return gf @ x2_hat.float().transpose(-2, -1), x1_hat.float().transpose(-2, -1) @ gf


# --------------------------------------------------------------------------------------
# NF4 frozen base weights           call sites: bitsandbytes_fix/_function.py:509, :540
# --------------------------------------------------------------------------------------
# bitsandbytes (unpinned fork, README.md:37-49) is neither vendored by the reference nor installed, so this is a
# restatement of its published NF4 block format: PARITY UNPINNED by reference outputs.
NF4_LEVELS = torch.tensor([
    -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
    -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
    0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941, 0.7229568362236023,
    1.0], dtype=torch.float32)


def nf4_quantize(w, block=64):
    """-> (packed uint8 [n/2], absmax fp32 [n/block]).  v = w * (1/absmax) in fp32; level index = number of
    midpoints between neighbouring levels strictly below v; first weight of a pair in the high nibble."""
    flat = w.float().reshape(-1, block)
    absmax = flat.abs().amax(dim=1)
    inv = torch.where(absmax > 0, 1.0 / absmax, torch.zeros_like(absmax))
    v = flat * inv[:, None]
    mids = 0.5 * (NF4_LEVELS[:-1] + NF4_LEVELS[1:])
    codes = (v[..., None] > mids).sum(-1).to(torch.uint8).reshape(-1, 2)
    return (codes[:, 0] << 4) | codes[:, 1], absmax


def nf4_dequantize(packed, absmax, shape, block=64):
    codes = torch.stack([packed >> 4, packed & 15], dim=1).reshape(-1, block).long()
    return (NF4_LEVELS[codes] * absmax[:, None]).to(BF16).reshape(shape)


# --------------------------------------------------------------------------------------
# rotary position embedding                       models/modeling_llama.py:229-260
# --------------------------------------------------------------------------------------
def rotate_half(x):
    """models/modeling_llama.py:229-233"""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def rope_fwd(x, cos, sin):
    """x [B, nh, S, hd], cos / sin [S, hd] -> x*cos + rotate_half(x)*sin (models/modeling_llama.py:258-259), in fp32
    with one rounding to x's dtype (the reference rounds each of its three bf16 steps)"""
    xf = x.float()
    return (xf * cos.float() + rotate_half(xf) * sin.float()).to(x.dtype)


def rope_bwd(g, cos, sin):
    """transpose of rope_fwd: d/dx of sum(g * rope_fwd(x))"""
    gf = g.float()
    return (gf * cos.float() - rotate_half(gf * sin.float())).to(g.dtype)


# --------------------------------------------------------------------------------------
# seeded dropout                                  operators/efficient_dropout.py:7-79
# --------------------------------------------------------------------------------------
# The reference's kernels are Triton (cannot run without a GPU) and draw their mask with tl.rand; this restates
# triton/language/random.py of the installed triton 3.6.0 (the reference pins no version): Philox4x32-10 with counter
# (index, 0, 0, 0) and key (seed & 0xffffffff, seed >> 32), first output word, folded to a non-negative int32 and
# scaled by 4.6566127342e-10.  PARITY UNPINNED by reference outputs; the generator is pinned by the Random123
# known-answer vectors.
def philox4x32_10(counter, key):
    """counter: four uint32 arrays (or ints), key: two -> four uint32 arrays; numpy uint64 arithmetic"""
    import numpy as np
    c0, c1, c2, c3 = (np.asarray(c, dtype=np.uint64) for c in counter)
    k0, k1 = (np.uint64(k) for k in key)
    A, B, M = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57), np.uint64(0xFFFFFFFF)
    for _ in range(10):
        pa, pb = A * c0, B * c2
        c0, c1, c2, c3 = ((pb >> np.uint64(32)) ^ c1 ^ k0) & M, pb & M, ((pa >> np.uint64(32)) ^ c3 ^ k1) & M, pa & M
        k0, k1 = (k0 + np.uint64(0x9E3779B9)) & M, (k1 + np.uint64(0xBB67AE85)) & M
    return c0, c1, c2, c3


def dropout_keep_mask(n, p, seed):
    """bool [n]: tl.rand(seed, i) > p for i in 0..n-1 (operators/efficient_dropout.py:24-25)"""
    import numpy as np
    idx = np.arange(n, dtype=np.uint64)
    zero = np.zeros(n, dtype=np.uint64)
    word = philox4x32_10((idx, zero, zero, zero), (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))[0].astype(np.uint32)
    v = word.view(np.int32).astype(np.int64)
    v = np.where(v < 0, -v - 1, v)
    u = v.astype(np.float32) * np.float32(4.6566127342e-10)
    return torch.from_numpy(u > np.float32(p))


def dropout_fwd(x, p, seed):
    """where(keep, x / (1 - p), 0) (:27): fp32 division, rounded to x's dtype"""
    keep = dropout_keep_mask(x.numel(), p, seed).reshape(x.shape)
    scaled = (x.float() / torch.tensor(1.0, dtype=torch.float32).sub(torch.tensor(p, dtype=torch.float32))).to(x.dtype)
    return torch.where(keep, scaled, torch.zeros_like(x))


def dropout_bwd(g, p, seed):
    """where(keep, g, 0) (:52): the reference does not rescale the gradient"""
    keep = dropout_keep_mask(g.numel(), p, seed).reshape(g.shape)
    return torch.where(keep, g, torch.zeros_like(g))
