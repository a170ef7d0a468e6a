"""Host-side mirror of the reference's operators/compress_function.py: same function names, argument meaning
and return types, with the compress / decompress work done by the HIP kernels.

Calibration (get_statistics*) runs twice per module lifetime and is written with torch device ops; everything
that runs every step goes through the C ABI.  Inputs must live on the GPU: there is no CPU path.
"""
import torch

from .. import kernels as K

BF16 = torch.bfloat16


# ---- shape helpers (reference: operators/compress_function.py:4-12) --------------------------------------
def hidden_to_head_shape(x: torch.Tensor, num_heads: int):
    b, s, h = x.shape
    return x.reshape(b, s, num_heads, h // num_heads).transpose(1, 2)


def head_to_hidden_shape(x: torch.Tensor):
    b, nh, s, hd = x.shape
    return x.transpose(1, 2).reshape(b, s, nh * hd)


@torch.no_grad()
def pad_cut_L(src_L, tgt_L):
    """rows of src_L padded with zeros / cut to the row count of tgt_L (reference :350-360)"""
    return K.fit_rows(src_L, tgt_L.shape[0])


# ---- calibration (reference :292-347) ------------------------------------------------------------------------
@torch.no_grad()
def get_statistics(x: torch.Tensor, iteration: int, outlier_ratio: float, sub_outlier_ratio: float,
                   sub_outlier_bit: int = 8, sub_outlier_quantize_method: str = 'per-tensor', svd_rank: int = 16):
    """(threshold fp32 0-d, L bf16 [S,r], R bf16 [r,H], scale bf16) from batch element 0"""
    if x.dim() == 4:
        x = head_to_hidden_shape(x)
    S, H = x.shape[-2], x.shape[-1]
    if svd_rank > 0:
        U, sv, V = torch.svd_lowrank(x[0].to(torch.float32), q=svd_rank, niter=16)
        L = U.contiguous()
        R = (torch.diag(sv) @ V.T).contiguous()
        x = x - L @ R
    else:
        L = torch.zeros((S, 16), dtype=x.dtype, device=x.device)
        R = torch.zeros((16, H), dtype=x.dtype, device=x.device)
    x0 = x[0]
    kth = int(x0.numel() * (1 - outlier_ratio))
    outlier = K.kth_value(x0, kth)
    x = x - (x0 * (x0.abs() > outlier)).to(BF16)
    if sub_outlier_ratio > 0 and sub_outlier_bit != 16:
        z = x[0]
        levels = 2 ** sub_outlier_bit - 1
        if sub_outlier_quantize_method == 'per-tensor':
            scale = (z.max() - z.min()) / levels
        elif sub_outlier_quantize_method == 'per-channel':
            scale = (z.amax(dim=-2, keepdim=True) - z.amin(dim=-2, keepdim=True)) / levels
        elif sub_outlier_quantize_method == 'per-token':
            scale = (z.amax(dim=-1, keepdim=True) - z.amin(dim=-1, keepdim=True)) / levels
        else:
            raise ValueError("Unsupport Quantize Method")
    else:
        scale = torch.tensor(1., device=x.device)
    return outlier, L.to(BF16), R.to(BF16), scale.to(BF16)


@torch.no_grad()
def get_statistics_softmax(x: torch.Tensor, iteration: int, outlier_ratio: float):
    x0 = x[0]
    return K.kth_value(x0, int(x0.numel() * (1 - outlier_ratio)))


# ---- compress / decompress (reference :136-261) --------------------------------------------------------------
def _check_quantised(sub_outlier_bit, sub_outlier_ratio):
    if sub_outlier_ratio == 0.:
        raise NotImplementedError("sub_outlier_ratio == 0 (no quantised part) is outside the accelerated path")
    assert (sub_outlier_bit in [1, 2, 4, 8, 16]), "Only support 1,2,4,8,16 bit quantization"
    if sub_outlier_bit == 16:
        raise NotImplementedError("sub_outlier_bit == 16 (no quantisation) is outside the accelerated path")


def compress_to_csr(x, outlier, scale, sub_outlier_bit, sub_outlier_ratio, L, R, exact=False):
    """the kernels' own container (codes + CSR outliers); x is [B,S,H] or [B,nh,S,hd].  exact: size the outlier arrays by
    reading their total back (what a conversion to COO needs); otherwise a frozen threshold tensor sizes them ahead
    of time from its second use on (kernels.KeptBudget)."""
    _check_quantised(sub_outlier_bit, sub_outlier_ratio)
    if x.dim() == 4:
        x = head_to_hidden_shape(x)
    x = x.contiguous()
    S, H = x.shape[-2], x.shape[-1]
    rank0 = L is None or not bool(L.shape[-1]) or (L.shape[-1] == 16 and getattr(L, "_hyc_zero", False))
    c = K.compress_threshold(x.reshape(-1, H), S, K.threshold_value(outlier), scale.contiguous(), sub_outlier_bit,
                             None if rank0 else L.contiguous(), None if rank0 else R.contiguous(),
                             budget=None if exact else K.kept_budget(outlier))
    return c, tuple(x.shape)


def csr_to_coo(c, shape):
    """CSR outliers -> the sparse COO tensor `.to_sparse()` gives in the reference (int64 indices, row-major)"""
    S = shape[-2]
    counts = (c.row_ptr[1:] - c.row_ptr[:-1]).long()
    rows = torch.repeat_interleave(torch.arange(c.M, device=counts.device), counts)
    lead = [rows]
    if len(shape) == 3:
        lead = [rows // S, rows % S]
    idx = torch.stack(lead + [c.cols.long()])
    return torch.sparse_coo_tensor(idx, c.vals, shape, is_coalesced=True)


def coo_to_csr(coo, M, S):
    coo = coo.coalesce()
    idx = coo.indices()
    rows = idx[0] * S + idx[1] if idx.shape[0] == 3 else idx[0]
    row_ptr = torch.zeros(M + 1, dtype=torch.int32, device=idx.device)
    if rows.numel():
        torch.cumsum(torch.bincount(rows, minlength=M), 0, out=row_ptr[1:])
    return row_ptr, idx[-1].to(torch.int32).contiguous(), coo.values().to(BF16).contiguous()


@torch.no_grad()
def true_divide_outlier_suboutlier_svd_compress(x: torch.Tensor, outlier: float, scale: float, sub_outlier_bit: int = 8,
                                                sub_outlier_ratio: float = 1., L: torch.Tensor = None,
                                                R: torch.Tensor = None):
    """-> (outliers as a sparse COO bf16 tensor, packed codes [B,S,H*bit/8] uint8 (int8 [B,S,H] for 8 bits), scale)"""
    c, shape = compress_to_csr(x, outlier, scale, sub_outlier_bit, sub_outlier_ratio, L, R, exact=True)
    return csr_to_coo(c, shape), c.stored.reshape(shape[:-1] + (c.stored.shape[-1],)), scale


@torch.no_grad()
def true_divide_outlier_suboutlier_svd_decompress(x_outlier_compressed, x_sub_outlier_compressed, sub_outlier_bit, scale,
                                                  is_head=False, num_heads=1, L=None, R=None):
    shape = tuple(x_outlier_compressed.shape)
    S, H = shape[-2], shape[-1]
    M = 1
    for d in shape[:-1]:
        M *= d
    row_ptr, cols, vals = coo_to_csr(x_outlier_compressed, M, S)
    rank0 = L is None or not bool(L.shape[-1])
    Lf = None if rank0 else K.fit_rows(L.contiguous(), S)
    c = K.ThresholdCompressed(x_sub_outlier_compressed.reshape(M, -1).contiguous(), row_ptr, cols, vals,
                              0.0, scale.contiguous(), Lf, None if rank0 else R.contiguous(), sub_outlier_bit, M, H, S)
    x = K.decompress_threshold(c).reshape(shape)
    if is_head:
        x = hidden_to_head_shape(x, num_heads=num_heads)
    return x


# ---- softmax sparsification (reference :264-281) -----------------------------------------------------------
def prune_softmax(x: torch.Tensor, outlier: float):
    return K.softmax_prune(x, outlier)


@torch.no_grad()
def true_compress_softmax(x: torch.Tensor, outlier: float):
    """probabilities above the threshold as a sparse COO tensor (same indices / values as `.to_sparse()`)"""
    return K.softmax_sparse_coo(x, outlier)


@torch.no_grad()
def true_decompress_softmax(x_sparse: torch.Tensor):
    return K.sparse_coo_to_dense(x_sparse)


# ---- small helpers other code may import (reference :71-95, :284-290) -------------------------------------
def convert_coo_to_tuple(x_coo):
    """identity, as in the reference (its int16 tuple form sits unreachable behind an early return)"""
    return x_coo


def convert_tuple_to_coo(x_coo_tuple):
    return x_coo_tuple


def profile_memory(name):
    """debug print of the allocator state in MiB"""
    mib = 1024 * 1024
    print("%s %s %s" % ("-" * 21, name, "-" * 21))
    print("allocated: %.2f MB" % (torch.cuda.memory_allocated() / mib), flush=True)
    print("reserved:  %.2f MB" % (torch.cuda.memory_reserved() / mib), flush=True)
    print("-" * 50)
