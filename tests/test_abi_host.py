"""CPU-only checks of the boundary: the shared library loads, exports every symbol include/hyc_abi.h declares,
rejects bad arguments with the documented codes without touching a GPU, and the host-side calibration logic
follows the reference's running-mean protocol."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from conftest import ROOT, bits_equal, from_bits


@pytest.fixture(scope="module")
def abi(hyc):
    if not os.path.exists(hyc._abi.LIB_PATH):
        pytest.skip("library not built (python hyc-lora_amd/build.py)")
    return hyc._abi


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "hyc_abi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hyc_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(abi):
    lib = abi.load()
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), n
        assert n in abi.SIGNATURES, "no ctypes prototype for " + n
    assert sorted(abi.SIGNATURES) == names
    assert lib.hyc_abi_version() == 3


def test_desc_layout_matches_header(abi):
    d = abi.HycDesc
    assert (d.mode.offset, d.bits.offset, d.group.offset, d.k.offset) == (0, 4, 8, 12)
    assert d.chan_plan.offset == 16 and d.threshold.offset == 24 and d.scale.offset == 32
    assert d.scale_stride_token.offset == 40 and d.S.offset == 56 and d.L.offset == 64 and d.rank.offset == 80
    assert d.csr_row_ptr.offset == 88 and d.chan_idx.offset == 112 and ctypes.sizeof(d) == 120


def test_shape_queries(abi):
    lib = abi.load()
    assert lib.hyc_check_shape(4096, 4, 128, abi.MODE_CHANNEL) == 0
    assert lib.hyc_check_shape(11008, 2, 64, abi.MODE_CHANNEL) == 0
    assert lib.hyc_check_shape(4100, 4, 128, abi.MODE_CHANNEL) == abi.ENOTSUP
    assert b"multiple of 16" in lib.hyc_last_error()
    assert lib.hyc_check_shape(4096, 3, 128, abi.MODE_CHANNEL) == abi.ENOTSUP
    assert lib.hyc_check_shape(4096, 4, 96, abi.MODE_CHANNEL) == abi.ENOTSUP
    assert lib.hyc_check_shape(4096, 4, 0, abi.MODE_THRESHOLD) == 0
    assert lib.hyc_check_shape(0, 4, 128, abi.MODE_CHANNEL) == abi.EINVAL
    assert lib.hyc_check_shape(4096, 4, 128, 7) == abi.EINVAL
    assert lib.hyc_stored_row_bytes(4096, 4) == 2048 and lib.hyc_stored_row_bytes(11008, 2) == 2752
    assert lib.hyc_rmsnorm_bwd_partials(0, 4096) == 0 and lib.hyc_rmsnorm_bwd_partials(4096, 4096) >= 1
    assert lib.hyc_gradw_workspace_bytes(4096, 4096, 4096) == 0
    assert lib.hyc_gradw_workspace_bytes(4096, 16, 4096) % (16 * 4096 * 4) == 0


def test_argument_errors_without_a_gpu(abi):
    """every entry point validates before it launches: these calls return before any HIP call is made"""
    lib = abi.load()
    d = abi.HycDesc()
    d.mode, d.bits, d.group, d.k = abi.MODE_CHANNEL, 4, 128, 0
    null = None
    assert lib.hyc_compress(null, 4, 4096, None, null, null, null, null, null) == abi.EFAULT
    assert lib.hyc_compress(null, 4, 4096, ctypes.byref(d), null, null, null, null, null) == abi.EFAULT      # no plan
    d.chan_plan = 0x1000
    assert lib.hyc_compress(null, 4, 4096, ctypes.byref(d), null, null, null, null, null) == abi.EFAULT      # null x
    assert lib.hyc_compress(null, -1, 4096, ctypes.byref(d), null, null, null, null, null) == abi.EINVAL
    assert lib.hyc_compress(null, 0, 4096, ctypes.byref(d), null, null, null, null, null) == 0               # empty input
    assert lib.hyc_compress(0x1001, 4, 4096, ctypes.byref(d), 0x2000, null, 0x3000, null, null) == abi.EINVAL  # misaligned
    d.bits = 3
    assert lib.hyc_decompress(null, null, null, 4, 4096, ctypes.byref(d), null, null) == abi.ENOTSUP
    d.bits = 4
    t = abi.HycDesc()
    t.mode, t.bits = abi.MODE_THRESHOLD, 8
    assert lib.hyc_rmsnorm_bwd(null, null, null, null, null, 0, null, 4, 4096, ctypes.byref(t), 1, null, null, 0x10, null) == abi.ENOTSUP
    assert lib.hyc_act_bwd(9, null, null, null, null, 4, 4096, ctypes.byref(d), null, null) == abi.EINVAL
    assert lib.hyc_gradw_gemm(null, 20, null, null, null, 4, 20, 4096, ctypes.byref(d), 1.0, 0.0, 0x10, 0, null, null) == abi.ENOTSUP
    assert lib.hyc_softmax_fwd(null, 4, 12, 0.0, 0x10, null, null) == abi.ENOTSUP
    assert lib.hyc_low_rank_update(null, null, null, null, 4, 0, 64, 2, 1, null) == abi.EINVAL
    assert lib.hyc_softmax_causal_fwd(null, 4, 8192, 4, 0.0, null, null, null) == abi.ENOTSUP
    assert lib.hyc_softmax_causal_fwd(null, 4, 64, 0, 0.0, null, null, null) == abi.EINVAL
    assert lib.hyc_softmax_causal_fwd(null, 4, 64, 65, 0.0, null, null, null) == abi.EINVAL
    assert lib.hyc_softmax_causal_fwd(null, 4, 64, 4, 0.0, null, null, null) == abi.EFAULT
    assert lib.hyc_rope_to_heads(null, 96, null, null, 2, 8, 4, 24, null, null, null) == abi.EINVAL      # head_dim % 16
    assert lib.hyc_rope_to_heads(null, 128, null, null, 0, 8, 4, 32, null, null, null) == 0
    assert lib.hyc_rope_to_heads(null, 120, null, null, 2, 8, 4, 32, null, null, null) == abi.EINVAL     # pitch < heads*head_dim
    assert lib.hyc_rope_to_heads(null, 128, null, null, 2, 8, 4, 32, null, null, null) == abi.EFAULT
    assert lib.hyc_rope_from_heads(null, null, null, 2, 8, 0, 32, null, null) == abi.EINVAL
    assert lib.hyc_rope_from_heads(null, null, null, 1 << 20, 1 << 12, 64, 128, null, null) == abi.EINVAL   # 2^31 items
    assert lib.hyc_dropout(null, null, 16, 1.0, 5, 0, null) == abi.EINVAL              # p must be below 1
    assert lib.hyc_dropout(null, null, 1 << 31, 0.1, 5, 0, null) == abi.EINVAL
    assert lib.hyc_dropout(null, null, 0, 0.1, 5, 0, null) == 0
    assert lib.hyc_dropout(null, null, 16, 0.1, 5, 0, null) == abi.EFAULT
    assert lib.hyc_compress_rows(null, 4000, 4, 4096, ctypes.byref(d), null, null, null, null, null) == abi.EINVAL       # pitch < H
    assert lib.hyc_compress_rows(null, 4100, 4, 4096, ctypes.byref(d), null, null, null, null, null) == abi.EINVAL       # pitch % 8
    assert lib.hyc_compress_rows(null, 8192, 4, 4096, ctypes.byref(t), null, null, null, null, null) == abi.EINVAL  # threshold scheme
    assert lib.hyc_compress_rows(null, 8192, 4, 4096, ctypes.byref(d), null, null, null, null, null) == abi.EFAULT
    assert lib.hyc_kth_value_workspace_bytes() >= 1024 + 12
    assert lib.hyc_kth_value(null, 7, 10, 1, null, null, null) == abi.ENOTSUP
    assert lib.hyc_kth_value(null, abi.DTYPE_F32, 0, 1, null, null, null) == abi.EINVAL
    assert lib.hyc_kth_value(null, abi.DTYPE_F32, 10, 11, null, null, null) == abi.EINVAL
    assert lib.hyc_kth_value(null, abi.DTYPE_BF16, 10, 0, null, null, null) == abi.EINVAL
    assert lib.hyc_kth_value(null, abi.DTYPE_BF16, 10, 3, null, null, null) == abi.EFAULT
    assert lib.hyc_nf4_quantize(null, 100, null, null, null) == abi.EINVAL            # not a multiple of 64
    assert lib.hyc_nf4_quantize(null, 0, null, null, null) == 0
    assert lib.hyc_nf4_quantize(null, 128, null, null, null) == abi.EFAULT
    assert lib.hyc_nf4_dequantize(null, null, -64, null, null) == abi.EINVAL
    assert lib.hyc_nf4_dequantize(null, null, 64, null, null) == abi.EFAULT
    assert lib.hyc_select_channels(null, 4096, 5000, null, null, null) == abi.EINVAL
    # the entry points added on top of the reference's operator set
    D = ctypes.byref(d)
    assert lib.hyc_gated_act_bwd(9, null, null, null, null, D, null, null, null, D, null, null, null, D, 4, 4096, null, null, null) == abi.EINVAL
    assert lib.hyc_gated_act_bwd(abi.ACT_SILU, null, null, null, null, D, null, null, null, D, null, null, null, ctypes.byref(t),
                                 4, 4096, null, null, null) == abi.ENOTSUP                                   # not channel-compressed
    d2 = abi.HycDesc()
    d2.mode, d2.bits, d2.group, d2.k, d2.chan_plan = abi.MODE_CHANNEL, 2, 64, 0, 0x1000
    assert lib.hyc_gated_act_bwd(abi.ACT_SILU, null, null, null, null, D, null, null, null, ctypes.byref(d2), null, null, null, D,
                                 4, 4096, null, null, null) == abi.ENOTSUP                                   # mixed code widths
    assert lib.hyc_gated_act_bwd(abi.ACT_SILU, null, null, null, null, D, null, null, null, D, null, null, null, D,
                                 4, 4096, null, null, null) == abi.EFAULT                                    # null buffers
    assert lib.hyc_gated_act_bwd(abi.ACT_SILU, null, null, null, null, D, null, null, null, D, null, null, null, D,
                                 0, 4096, null, null, null) == 0                                             # empty input
    nine = [null] * 9
    assert lib.hyc_gated_act_fwd(9, null, 4096, null, 4096, 4, 4096, D, D, D, null, *nine, null) == abi.EINVAL
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 4096, null, 4096, 4, 4096, D, D, ctypes.byref(t), null, *nine, null) == abi.ENOTSUP
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 4096, null, 4096, 4, 4096, D, ctypes.byref(d2), D, null, *nine, null) == abi.ENOTSUP
    d2b = ctypes.byref(d2)
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 4096, null, 4096, 4, 4096, d2b, d2b, d2b, null, *nine, null) == abi.EFAULT   # 2-bit codes: covered
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 20480, null, 20480, 4, 20480, d2b, d2b, d2b, null, *nine, null) == abi.EFAULT   # 640 chunks: two parts of 320
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 32832, null, 32832, 4, 32832, d2b, d2b, d2b, null, *nine, null) == abi.ENOTSUP  # 1026 chunks: row too long
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 14336, null, 14336, 4, 14336, D, D, D, null, *nine, null) == abi.EFAULT     # 896 chunks: two workgroups per row
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 13824, null, 13824, 4, 13824, D, D, D, null, *nine, null) == abi.EFAULT     # 864 chunks: two parts of 27 groups
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 12544, null, 12544, 4, 12544, D, D, D, null, *nine, null) == abi.ENOTSUP    # 784 chunks = 49 groups: no 2 to 4 equal parts
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 4000, null, 4096, 4, 4096, D, D, D, null, *nine, null) == abi.EINVAL   # pitch < H
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 8192, null, 4100, 4, 4096, D, D, D, null, *nine, null) == abi.EINVAL   # pitch % 8
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 8192, null, 8192, 4, 4096, D, D, D, null, *nine, null) == abi.EFAULT
    assert lib.hyc_gated_act_fwd(abi.ACT_GELU_TANH, null, 8192, null, 8192, 0, 4096, D, D, D, null, *nine, null) == 0
    assert lib.hyc_gated_act_fwd(abi.ACT_SILU, null, 65536, null, 65536, 4, 65536, D, D, D, null, *nine, null) == abi.ENOTSUP  # row too long
    six = [null] * 6
    assert lib.hyc_act_fwd_compress(9, null, 4096, 4, 4096, D, null, null, null, null, null) == abi.EINVAL
    assert lib.hyc_act_fwd_compress(abi.ACT_SILU, null, 4096, 4, 4096, None, null, null, null, null, null) == abi.EFAULT
    assert lib.hyc_act_fwd_compress(abi.ACT_SILU, null, 4096, 4, 4096, ctypes.byref(t), null, null, null, null, null) == abi.ENOTSUP
    assert lib.hyc_act_fwd_compress(abi.ACT_SILU, null, 4000, 4, 4096, D, null, null, null, null, null) == abi.EINVAL
    assert lib.hyc_act_fwd_compress(abi.ACT_GELU_TANH, null, 4096, 4, 4096, D, null, null, null, null, null) == abi.EFAULT
    assert lib.hyc_act_fwd_compress(abi.ACT_GELU_TANH, null, 4096, 0, 4096, D, null, null, null, null, null) == 0
    assert lib.hyc_hadamard_fwd_compress(null, 4096, null, 4096, 4, 4096, D, None, null, *six, null) == abi.EFAULT
    assert lib.hyc_hadamard_fwd_compress(null, 4096, null, 4096, 4, 4096, D, ctypes.byref(d2), null, *six, null) == abi.ENOTSUP
    assert lib.hyc_hadamard_fwd_compress(null, 4096, null, 4096, 4, 4096, d2b, d2b, null, *six, null) == abi.EFAULT    # two 2-bit operands: covered
    assert lib.hyc_hadamard_fwd_compress(null, 20480, null, 20480, 4, 20480, d2b, d2b, null, *six, null) == abi.ENOTSUP  # ... to 512 chunks
    assert lib.hyc_hadamard_fwd_compress(null, 4096, null, 4100, 4, 4096, D, D, null, *six, null) == abi.EINVAL
    assert lib.hyc_hadamard_fwd_compress(null, 4096, null, 4096, 4, 4096, D, D, null, *six, null) == abi.EFAULT
    assert lib.hyc_layernorm_fwd_compress(null, null, null, 0, 1e-5, 4, 4096, None, null, null, null, null, null, null, null, null) == abi.EFAULT
    assert lib.hyc_layernorm_fwd_compress(null, null, null, 7, 1e-5, 4, 4096, D, null, null, null, null, null, null, null, null) == abi.EINVAL
    assert lib.hyc_layernorm_fwd_compress(null, null, null, 0, 1e-5, 4, 4096, D, null, null, null, null, null, null, null, null) == abi.EFAULT
    assert lib.hyc_layernorm_fwd_compress(null, null, null, 0, 1e-5, 0, 4096, D, null, null, null, null, null, null, null, null) == 0
    assert lib.hyc_layernorm_fwd_compress(null, null, null, 0, 1e-5, 4, 32768, D, null, null, null, null, null, null, null, null) in (abi.EFAULT, abi.ENOTSUP)
    assert lib.hyc_layernorm_bwd(null, null, null, null, null, 0, null, null, 4, 4096, D, null, null, null, null) == abi.EFAULT
    assert lib.hyc_layernorm_bwd(null, null, null, null, null, 0, null, null, 4, 4096, ctypes.byref(t), null, null, null, null) in (abi.EFAULT, abi.ENOTSUP)
    assert lib.hyc_rmsnorm_bwd_partial_rows(0, 4096, D) == 0
    rows = lib.hyc_rmsnorm_bwd_partial_rows(4096, 4096, D)
    assert 1 <= rows <= lib.hyc_rmsnorm_bwd_partials(4096, 4096)
    assert lib.hyc_gradw_workspace_bytes(4096, 16, 4096) >= 2 * 16 * 4096 * 4          # the LoRA-A shape splits the tokens
    with pytest.raises(NotImplementedError):
        abi.check(abi.ENOTSUP)
    with pytest.raises(ValueError):
        abi.check(abi.EINVAL)


def test_launchers_refuse_cpu_tensors(hyc, abi):
    K = hyc.kernels
    with pytest.raises(ValueError, match="CUDA"):
        K.channel_absmax(torch.zeros(4, 64, dtype=torch.bfloat16))
    assert K.num_outlier_channels(4096, 0.01) == 41 and K.num_outlier_channels(11008, 0.01) == 110
    assert K.num_outlier_channels(4096, 0.005) == 20
    assert K.scale_strides(torch.zeros(()), 16, 64) == (0, 0)
    assert K.scale_strides(torch.zeros(1, 64), 16, 64) == (0, 1)
    assert K.scale_strides(torch.zeros(16, 1), 16, 64) == (1, 0)
    with pytest.raises(ValueError):
        K.scale_strides(torch.zeros(3, 5), 16, 64)


def test_running_mean_protocol_against_reference(hyc, golden_modules):
    """fold_statistics (host logic of every module) reproduces the reference modules' static values after calls 0
    and 1 when fed the per-call statistics the reference computed"""
    from oracle import hyc_oracle as O
    fold = hyc.operators._calibration.fold_statistics
    gm = golden_modules
    tag = "silu_b8_pt_r2"
    static = [None] * 4
    for call in range(2):
        p = f"{tag}_call{call}_"
        x = from_bits(gm[p + "x0"])
        torch.manual_seed(900 + call)
        thr, L, R, scale = O.get_statistics(x, call, 0.05, 1.0, 8, 'per-token', 2)
        static = fold(static, call, thr, L, scale, R)
        assert torch.equal(static[0], from_bits(gm[p + "s0_thr"]))
        assert bits_equal(static[1], from_bits(gm[p + "s0_L"])) and bits_equal(static[3], from_bits(gm[p + "s0_R"]))
        assert bits_equal(static[2], from_bits(gm[p + "s0_scale"]))


def test_module_constructors_mirror_the_reference(hyc):
    ops = hyc.operators
    m = ops.EfficientMemoryRMSNorm(64, eps=1e-6, elementwise_affine=True, bias=False, outlier_ratio=0.005,
                                   sub_outlier_ratio=1.0, sub_outlier_bit=8, sub_outlier_quantize_method='per-channel', rank=2)
    assert isinstance(m, torch.nn.LayerNorm) and m.iteration == 0 and m.static_value == [None] * 4 and m.bias is None
    l = ops.EfficientMemoryLinear(128, 16, bias=False, outlier_ratio=0.01, sub_outlier_ratio=1.0, sub_outlier_bit=2,
                                  sub_outlier_quantize_method='per-token', rank=0)
    assert isinstance(l, torch.nn.Linear) and l.weight.shape == (16, 128)
    for cls in (ops.EfficientMemorySiLU, ops.EfficientMemoryGELU):
        a = cls(outlier_ratio=0.01, sub_outlier_ratio=0.2, sub_outlier_bit=8, sub_outlier_quantize_method='per-tensor', rank=16)
        assert a.iteration == 0 and a.static_value == [None] * 4
    s = ops.EfficientMemorySoftmax(outlier_ratio=0.05)
    assert s.static_value is None and s.outlier_ratio == 0.05
    dr = ops.EfficientMemoryDropout(0.1)
    assert dr.p == 0.1 and 0 <= dr.seed < 2 ** 32 and dr.training
    h = ops.EfficientMemoryHadamard()
    assert h.static_value_1 == [None] * 4 and h.sub_outlier_bit_2 == 8
    g1 = ops.EfficientMemoryGEMM(outlier_ratio_1=0.01, sub_outlier_ratio_1=0.2, sub_outlier_bit_1=8,
                                 sub_outlier_quantize_method_1='per-tensor', outlier_ratio_2=0.01, sub_outlier_ratio_2=0.2,
                                 sub_outlier_bit_2=4, sub_outlier_quantize_method_2='per-tensor', rank=16)
    assert g1.static_value_1 == [None] * 4 and g1.static_value_2 == [None] * 4 and g1.sub_outlier_bit_2 == 4
    g2 = ops.EfficientMemoryGEMMWithSoftmax(outlier_ratio_1=0.05, outlier_ratio_2=0.01, sub_outlier_ratio_2=0.2,
                                            sub_outlier_bit_2=8, sub_outlier_quantize_method_2='per-tensor', rank=16)
    assert g2.static_value_1 is None and g2.static_value_2 == [None] * 4 and g2.iteration == 0
    fa = ops.EfficientFlashAttnVarlenQKVPacked(outlier_ratio=0.01, sub_outlier_ratio=0.2, sub_outlier_bit=8,
                                               sub_outlier_quantize_method='per-tensor', rank=16)
    assert fa.iteration == 0 and all(getattr(fa, n + "_static_value") == [None] * 4 for n in "qkvo")
    with pytest.raises(ValueError):
        ops.EfficientMemorySiLU(mode="bogus")
    cf = ops.compress_function
    for name in ("true_divide_outlier_suboutlier_svd_compress", "true_divide_outlier_suboutlier_svd_decompress",
                 "true_compress_softmax", "true_decompress_softmax", "prune_softmax", "get_statistics",
                 "get_statistics_softmax", "pad_cut_L", "hidden_to_head_shape", "head_to_hidden_shape",
                 "convert_coo_to_tuple", "convert_tuple_to_coo", "profile_memory"):
        assert callable(getattr(cf, name))
    assert callable(ops.fused_compression.low_rank_extraction) and callable(ops.fused_compression.low_rank_addition)
    x = torch.arange(2 * 3 * 8, dtype=torch.float32).reshape(2, 3, 8)
    assert torch.equal(cf.head_to_hidden_shape(cf.hidden_to_head_shape(x, 2)), x)


def test_module_swap_follows_the_reference_rules(hyc):
    """replace_module_for_quantization (train_gsm8k.py:426-592): trainable wide Linear, SiLU, RMSNorm, Softmax are
    swapped with their weights shared; frozen / narrow Linear and lm_head are not"""
    import torch
    ops = hyc.operators

    class TinyRMSNorm(torch.nn.Module):
        def __init__(self, h):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.ones(h))
            self.variance_epsilon = 1e-6

    class PlainGEMM(torch.nn.Module):
        def forward(self, a, b):
            return a @ b

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.norm = TinyRMSNorm(128)
            self.gemm1 = PlainGEMM()
            self.gemm2 = PlainGEMM()
            self.lora_A = torch.nn.Linear(128, 16, bias=False)
            self.lora_B = torch.nn.Linear(16, 128, bias=False)          # in_features <= 100: untouched
            self.base = torch.nn.Linear(128, 128)
            self.base.weight.requires_grad_(False)                      # frozen: untouched
            self.act_fn = torch.nn.SiLU()
            self.softmax = torch.nn.Softmax(dim=-1)
            self.drop = torch.nn.Dropout(0.1)
            self.lm_head = torch.nn.Linear(128, 128)

    model = torch.nn.Sequential(Block(), Block())
    cfg = {k: dict(outlier_ratio=0.01, sub_outlier_ratio=1.0, rank=0, sub_outlier_bit=4, sub_outlier_quant_method="per-token")
           for k in ("linear", "silu", "layernorm", "hadamard", "gemm")}
    cfg["softmax"] = dict(outlier_ratio=0.05)
    w_before = model[0].lora_A.weight.data_ptr()
    ops.replace_module_for_quantization(model, cfg, mode="hyc", group_size=64)
    b = model[1]
    assert isinstance(b.lora_A, ops.EfficientMemoryLinear) and b.lora_A.mode == "hyc" and b.lora_A.group_size == 64
    assert b.lora_A.sub_outlier_bit == 4 and b.lora_A.rank == 0
    assert model[0].lora_A.weight.data_ptr() == w_before
    assert type(b.lora_B) is torch.nn.Linear and type(b.base) is torch.nn.Linear and type(b.lm_head) is torch.nn.Linear
    assert isinstance(b.norm, ops.EfficientMemoryRMSNorm) and b.norm.eps == 1e-6 and b.norm.bias is None
    assert isinstance(b.act_fn, ops.EfficientMemorySiLU) and isinstance(b.softmax, ops.EfficientMemorySoftmax)
    assert b.softmax.outlier_ratio == 0.05
    assert isinstance(b.gemm1, ops.EfficientMemoryGEMM) and b.gemm1.sub_outlier_bit_2 == 4 and b.gemm1.mode == "hyc"
    assert isinstance(b.gemm2, ops.EfficientMemoryGEMMWithSoftmax) and b.gemm2.outlier_ratio_1 == 0.05
    assert isinstance(b.drop, ops.EfficientMemoryDropout) and b.drop.p == 0.0          # sic: the reference swaps in p = 0

    class Args:
        model_name_or_path = "google/gemma-7b"
    gm = torch.nn.Sequential(Block())
    ops.replace_module_for_quantization(gm, cfg, Args())
    assert isinstance(gm[0].norm, ops.EfficientMemoryRMSNormGemma)
    import pytest
    ln = torch.nn.Sequential(torch.nn.LayerNorm(128, eps=1e-12))
    ops.replace_module_for_quantization(ln, cfg)
    assert isinstance(ln[0], ops.EfficientMemoryLayerNorm) and ln[0].eps == 1e-12


def test_calibration_state_round_trip(hyc, tmp_path):
    """calibration_state / load_calibration_state: iteration, static values and the channel plan survive torch.save,
    state_dict() is left alone, unknown names are reported"""
    import pytest
    import torch
    ops = hyc.operators
    K = hyc.kernels

    def build():
        return torch.nn.Sequential(ops.EfficientMemorySiLU(0.01, 1.0, 4, "per-token", 0, mode="hyc"),
                                   ops.EfficientMemorySoftmax(0.05),
                                   ops.EfficientMemoryHadamard(0.01, 1.0, 4, "per-token", 0.01, 1.0, 4, "per-token", 0),
                                   torch.nn.Linear(8, 8))
    src = build()
    src[0].iteration = 5
    src[0].site.amax = torch.arange(16, dtype=torch.float32)
    src[0].site.plan = K.ChannelPlan(16, 1, torch.tensor([15], dtype=torch.int32), torch.tensor([0, 7], dtype=torch.int32),
                                     "range")
    src[1].iteration, src[1].static_value = 2, torch.tensor(0.25)
    src[2].iteration = 2
    src[2].static_value_1 = [torch.tensor(1.5), torch.zeros(4, 16).bfloat16(), torch.ones(1, 8).bfloat16(), torch.zeros(16, 8).bfloat16()]
    state = ops.calibration_state(src)
    assert sorted(state) == ["0", "1", "2"]
    assert not any("static" in k or "extra" in k for k in src.state_dict())
    path = tmp_path / "calib.pt"
    torch.save(state, path)
    state = torch.load(path, weights_only=True)
    dst = build()
    if not torch.cuda.is_available():
        # the default target of a parameterless module is the current GPU: without one the call says so
        with pytest.raises(ValueError, match="device"):
            ops.load_calibration_state(build(), state)
    assert ops.load_calibration_state(dst, state, device="cpu") == []
    assert dst[0].site.plan.scale_rule == "range" and dst[0].site.plan.idx.device.type == "cpu"
    # a plan that stayed on the host is refused before any pointer reaches a kernel
    with pytest.raises(ValueError, match="CUDA"):
        K.channel_desc(dst[0].site.plan, 4, 16)
    with pytest.raises(ValueError, match="CUDA"):
        K.alloc_channel(2, 16, dst[0].site.plan, 4, 16, "cpu")
    assert dst[0].iteration == 5 and torch.equal(dst[0].site.amax, src[0].site.amax)
    assert dst[0].site.plan.k == 1 and torch.equal(dst[0].site.plan.idx, src[0].site.plan.idx)
    assert torch.equal(dst[0].site.plan.plan, src[0].site.plan.plan)
    assert dst[1].iteration == 2 and float(dst[1].static_value) == 0.25
    assert torch.equal(dst[2].static_value_1[2], src[2].static_value_1[2]) and dst[2].static_value_2 == [None] * 4
    assert dst[2].site_1.plan is None
    with pytest.raises(KeyError):
        ops.load_calibration_state(dst, {"nope": {"iteration": 1}})
    assert ops.load_calibration_state(dst, {"nope": {"iteration": 1}}, strict=False) == ["nope"]


def test_header_is_plain_c_and_links_from_a_c_program(abi, tmp_path):
    """The boundary is a C ABI: a C99 translation unit that includes only include/hyc_abi.h references every
    declared entry point, links against the library and gets the documented codes back (host-only calls)."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    names = declared_symbols()
    src = tmp_path / "host.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "hyc_abi.h"\n'
        "typedef void (*entry)(void);\n"
        "static const entry table[] = {\n" + "".join("  (entry)%s,\n" % n for n in names) + "};\n"
        "int main(void) {\n"
        "  hyc_desc d;\n"
        "  memset(&d, 0, sizeof d);\n"
        "  if (sizeof table / sizeof table[0] != %d) return 10;\n" % len(names) +
        "  if (hyc_abi_version() != HYC_ABI_VERSION) return 11;\n"
        "  if (hyc_check_shape(4096, 4, 128, HYC_MODE_CHANNEL) != HYC_OK) return 12;\n"
        "  if (hyc_check_shape(4100, 4, 128, HYC_MODE_CHANNEL) != HYC_ENOTSUP) return 13;\n"
        "  if (!strstr(hyc_last_error(), \"multiple of 16\")) return 14;\n"
        "  if (hyc_compress(0, 8, 4096, 0, 0, 0, 0, 0, 0) != HYC_EFAULT) return 15;\n"
        "  d.mode = HYC_MODE_CHANNEL; d.bits = 3; d.group = 128;\n"
        "  if (hyc_compress(0, 8, 4096, &d, 0, 0, 0, 0, 0) != HYC_ENOTSUP) return 16;\n"
        "  printf(\"%d entry points\\n\", (int)(sizeof table / sizeof table[0]));\n"
        "  return 0;\n}\n")
    exe = tmp_path / "host"
    libdir = os.path.dirname(abi.LIB_PATH)
    libname = os.path.basename(abi.LIB_PATH)[3:-3]
    cmd = [gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
           "-L", libdir, "-l" + libname, "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib",
           "-Wl,--allow-shlib-undefined"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert "%d entry points" % len(names) in r.stdout
